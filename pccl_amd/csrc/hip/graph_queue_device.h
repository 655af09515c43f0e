// graph_queue_device.h -- device side of the op-batching path: the control block and
// counters that live in the graph arena, and the persistent kernel that drains the ready
// queues.  The protocol is described at the top of graph_queue.hip, which holds the host
// side.  The kernel is instantiated per dtype in graph_queue_inst_*.hip so that the
// instances compile in parallel.
#pragma once

#include "plugin_common.h"
#include "reduce_copy_device.h"

namespace pccl_queue {

using namespace pccl_dev;

constexpr int kQueues = 8;  // one per XCD of an MI355X
constexpr unsigned int kDefaultSpinLimit = 2000000u;  // microseconds a wait inside the kernel may last

// Words that many workgroups update or poll, each alone on its 256-byte line.
// Device-scope atomics and sc1 loads are served at the memory side; an ordinary
// cached load of the same line parks a copy in an XCD's L2 that every later
// atomic must first probe out again.  Measured: with immutable fields (queue
// length, entry pointer, part count) sharing lines with ticket counters and
// dependency counts, a claim took 25 us and a part 13 us under 768 workgroups,
// against 1.7 us and 1.9 us with 64.  So: lines that are written during a run
// are touched by atomics / sc1 only, and everything a workgroup reads with
// ordinary loads lives on lines that no one writes during a run.
struct alignas(256) HotWord {
  unsigned int value;
};

// Device-resident control block; read-only during a run.  The reference's
// GraphBufferLayout is its first member, so the arena's base address is a
// GraphBufferLayout*.
struct GraphControl {
  pccl_graph_buffer_layout layout;
  pccl_operation_layout_header *headers;  // contiguous; layout.operators[i] == &headers[i]
  char *slots;                            // PayloadSlot of op i at slots + i * kPayloadStride
  const int *succ;                        // all successor uid lists, back to back
  HotWord *hot;                           // kHot* words, see below
  const int *group_base;                  // per op: first of its kPartGroups words in `groups`, or -1
  const int *entry_base;                  // per op: number of its part 0 (parts of an op are numbered in sequence)
  HotWord *groups;                        // part counters of the ops that count in groups, see finish_part
  HotWord *ready;                         // per op: dependencies that have arrived in this run
  unsigned long long *trace;              // null, or 4 words per queue entry (see kTrace*)
  unsigned int *part_arrivals;            // per queue entry (t * kQueues + q), 1 << part_shift words apart:
                                          // part-by-part dependencies that have arrived
  int part_shift;
  const int *succ_part_base;              // beside succ: entry index of part 0 of a successor released part by part
  const int *chain;                       // per op, kChainWords ints: see kChain* below
  const struct ForwardStep *chain_table;  // one row per op of every forward chain, chain after chain
  const struct SignalFuse *fuse;          // per op: the signal ops it carries
  int *queue_head[kQueues];               // &layout.ready_queues[q]->head_
  const unsigned long long *queue_entries[kQueues];
  const int *queue_count;                 // entries on each queue, then the mode word (1: no more entries than workgroups,
                                          // each workgroup takes the entry of its own number): in memory, not here, because which ops queue entries
                                          // (chains do not) can change with the operands' addresses, and what is in
                                          // this block is frozen into any launch that a stream capture has recorded
  unsigned int spin_limit;
  unsigned int n_ops;
  const struct WideEntry *wide_entries;   // a graph that runs as a wide launch: what workgroup b carries out (else null)
};

// One per workgroup of a wide launch (wide_body), in the order the entries were dealt in: the entry with
// everything that the drain kernel would fetch from the entry, the op's slot and its chain words one
// after the other, so that the payload is the first dependent load.  n == 0: nothing to do.
struct WideEntry {
  int uid;
  int n;           // elements of this part
  long lo;         // first element of this part
  int chain[4];    // the op's kChainWords words ({-1, 1, 0, 0} for an op outside any chain)
};
static_assert(sizeof(WideEntry) == 32, "wide entry size");

// An op of many parts does not count them on one word: atomics on one address are carried out
// one after the other (about 11 ns each), and 1024 parts of a 32 MiB op finishing within a few
// microseconds queued up behind each other (14 such ops took 690 us instead of 250).  Ops with
// more than kGroupThreshold parts count part p on group word p % kPartGroups (each alone on its
// line); the part that empties a group counts the group on the header's remaining_executors_,
// which for these ops starts at kPartGroups instead of required_executors_.
constexpr int kPartGroups = 8;
constexpr int kGroupThreshold = 16;

// Chains (ops that run behind another op in the same workgroup, part by part): per op
typedef int i32x4 __attribute__((ext_vector_type(4)));
constexpr int kChainWords = 4;
constexpr int kChainNext = 0;     // the op that runs behind this one, or -1
constexpr int kChainLength = 1;   // for the op a chain starts with: ops in it (1 for an op outside any chain)
constexpr int kChainForward = 2;  // head: 1 if the whole chain runs in one pass with values handed on in registers
                                  // (run_chain_forward); another op of such a chain: which of its inputs is the
                                  // previous op's output 0; an op of a chain that runs through memory: kChainFolded
                                  // if it is a COPY of the previous op's output 0 whose outputs that op stores itself
constexpr int kChainFolded = 2;
constexpr int kChainRow = 3;      // head of a forward chain: its first row in GraphControl::chain_table
constexpr int kMaxForwardSteps = 16;
// A queue entry: op uid | part << 32 | (op heads a chain) << 51.  The flag saves every other entry the
// load of its op's chain words.
constexpr int kMaxParts = 1 << 19;
constexpr unsigned long long kEntryChainHead = 1ull << 51;
// ... | (every part polls a signal word first) << 52: the op carries a GET_NOTIFIED (GraphControl::fuse; such an
// entry has the chain flag too, for the count of ops it stands for).
constexpr unsigned long long kEntryWaitsSignal = 1ull << 52;
// ... | (whoever completes the part stores the part's signal word) << 53: the op carries a NOTIFY of one word per part.
constexpr unsigned long long kEntryNotifiesPart = 1ull << 53;
// ... | (the part is not counted) << 54.  An op that nothing in the graph waits for, and that waits for no
// whole op itself (its arrivals word is never written, so there is nothing to put back), is not counted
// part by part: nobody would read the count.  Its completion is the run's: when every workgroup has left
// and none gave up, every entry has been carried out, and the last workgroup out reports all ops
// complete.  That takes one or two returning atomics out of the end of every workgroup whose last entry
// is such an op: all of them in graphs of independent ops and chains.
constexpr unsigned long long kEntryUncounted = 1ull << 54;
constexpr unsigned long long kEntryFlags = kEntryChainHead | kEntryWaitsSignal | kEntryNotifiesPart | kEntryUncounted;
// In a successor list: not an op, but "store the signal word of the NOTIFY this op carries".
constexpr int kSuccNotify = -1;

// indices into GraphControl::hot
constexpr int kHotCompleted = 0;  // *layout.completed_operator
constexpr int kHotTotal = 1;      // *layout.total_operator (never written during a run)
constexpr int kHotAbort = 2;      // set when a bounded wait gave up
constexpr int kHotExit = 3;       // 64 bits: workgroups that have left the current run | those that left a run given up << 16 | ops they completed << 32
constexpr unsigned int kExitQuit = 1u << 16;  // (a launch has fewer workgroups than that: graph_create checks)
constexpr int kHotRun = 4;        // number of the current run (first run = 1), bumped by the last workgroup out
constexpr int kHotWords = kHotRun + 1;

// What a workgroup needs to run a part, on lines nothing writes during a run: the
// op's payload plus the two header facts (part count, successor list) it would
// otherwise have to read from the header, whose line is under atomic fire.
constexpr size_t kPayloadStride = 256;
struct PayloadSlot {
  pccl_op_payload payload;  // 248 bytes; what OperationLayoutHeader::op_buffer_ points to
  int parts;                // == required_executors_
  int succ_start;           // successors at GraphControl::succ + succ_start
};
static_assert(sizeof(PayloadSlot) == kPayloadStride, "payload slot stride");

// What the bookkeeping of a finished part needs from the op's slot.  The workgroup reads it
// together with the payload when the part starts (uniform loads), so that no load stands
// between the end of the part and the atomics that hand it over.
struct OpFacts {
  int parts;
  int succ_start;
  unsigned int counts;  // payload bytes 4..7: pre_dependencies_, part_preds_, part_nexts_, num_next_ops_
  __device__ __forceinline__ static OpFacts of(const PayloadSlot *slot) {
    OpFacts f;
    f.parts = slot->parts;
    f.succ_start = slot->succ_start;
    f.counts = *(const unsigned int *)&slot->payload.pre_dependencies_;
    return f;
  }
  __device__ __forceinline__ int pre_dependencies() const { return (int)(counts & 0xffu); }
  __device__ __forceinline__ int part_preds() const { return (int)((counts >> 8) & 0xffu); }
  __device__ __forceinline__ int part_nexts() const { return (int)((counts >> 16) & 0xffu); }
  __device__ __forceinline__ int num_next_ops() const { return (int)(counts >> 24); }
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
    // Packs a lane has in flight: a part is short (8 packs per lane and stream at the built-in
    // part size), and every batch of loads costs a full memory latency before its stores can go.
    // (The variant for unaligned streams assembles each pack from two loads, and a pack of 8-bit
    // floats unpacks into 16 accumulators: both stay at 1-2 to keep three wavefronts per SIMD.)
    constexpr int kUnroll = !ALIGNED ? (NIN >= 3 ? 1 : 2) : NIN == 1 ? 4 : D::kElemBytes == 1 ? (NIN >= 3 ? 1 : 2) : NIN == 2 ? 4 : NIN <= 4 ? 2 : 1;
    body_packs<D, Op, NIN, kUnroll, ALIGNED, kMemCoherent, kMemCoherent>(body, n_packs, 0, 1);
  }
  if (threadIdx.x >= kBlock - kWave)
    edge_elems<D, Op, NIN, kMemCoherent>(a, head, head + n_packs * kEpp, count, (int)threadIdx.x - (kBlock - kWave));
  // (the caller waits for the stores where someone will read them during the run)
}

// SLIM: only the variant that tolerates unaligned streams (keeps the any-dtype instance small).
// `more`: null, or the payload of a COPY that is chained behind this op and whose input is this op's
// output 0 (kChainFolded): its outputs are stored by this op as further outputs, and the copy itself is
// not run.  The value goes from registers to every destination; nothing is written, waited for and read
// back between the two ops.
template <class D, class Op, int NIN, bool SLIM = false>
__device__ __forceinline__ void run_part_nin(const pccl_op_payload *pl, const pccl_op_payload *more, long lo, long count) {
  RcOperands a;
  const int own_out = pl->n_out_;
  a.n_out = own_out + (more ? more->n_out_ : 0);
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
      const void *to = j < own_out ? pl->chunks_[NIN + j].addr_ : more->chunks_[1 + j - own_out].addr_;
      a.out[j] = (char *)to + lo * D::kElemBytes;
      mis |= (unsigned long long)a.out[j] ^ (unsigned long long)a.out[0];
    }
  // same peel as the direct launch: make output 0 start on 16 bytes; the other
  // streams are 16-byte aligned after it exactly when they share its low bits
  long head = (long)((16 - ((unsigned long long)a.out[0] & 15)) & 15) / D::kElemBytes;
  if (head > count) head = count;
  const long n_packs = (count - head) / (16 / D::kElemBytes);
  const bool aligned = (mis & 15) == 0;
  if constexpr (SLIM) {
    run_part_body<D, Op, NIN, false>(a, head, n_packs, count);
  } else {
    if (aligned) run_part_body<D, Op, NIN, true>(a, head, n_packs, count);
    else run_part_body<D, Op, NIN, false>(a, head, n_packs, count);
  }
}

// COPY moves bytes, and its element size is its own, not that of the graph's REDUCE ops:
// it runs as a copy of 1-byte units.
__device__ __forceinline__ void run_copy_part(const pccl_op_payload *pl, const pccl_op_payload *more, long lo, long count) {
  const int dt = pl->chunks_[0].dtype_;
  const long units = dt == PCCL_F64 ? 8 : (dt == PCCL_F32 || dt == PCCL_I32 || dt == PCCL_U32) ? 4
                     : (dt == PCCL_BF16 || dt == PCCL_F16) ? 2 : 1;
  run_part_nin<Dtype<PCCL_F8E4M3>, OpSum, 1>(pl, more, lo * units, count * units);
}

template <int DT, class Op, bool SLIM = false>
__device__ __forceinline__ void run_reduce_part(const pccl_op_payload *pl, const pccl_op_payload *more, long lo, long count) {
  typedef Dtype<DT> D;
  switch (pl->n_in_) {
    case 2: run_part_nin<D, Op, 2, SLIM>(pl, more, lo, count); break;
    case 3: run_part_nin<D, Op, 3, SLIM>(pl, more, lo, count); break;
    case 4: run_part_nin<D, Op, 4, SLIM>(pl, more, lo, count); break;
    case 5: run_part_nin<D, Op, 5, SLIM>(pl, more, lo, count); break;
    case 6: run_part_nin<D, Op, 6, SLIM>(pl, more, lo, count); break;
    case 7: run_part_nin<D, Op, 7, SLIM>(pl, more, lo, count); break;
    default: run_part_nin<D, Op, 8, SLIM>(pl, more, lo, count); break;
  }
}

template <int DT, class Op>
__device__ __forceinline__ void run_part(const pccl_op_payload *pl, const pccl_op_payload *more, long lo, long count) {
  if (pl->n_in_ == 1) run_copy_part(pl, more, lo, count);
  else run_reduce_part<DT, Op>(pl, more, lo, count);
}

// A graph whose REDUCE ops do not share one (dtype, compute) pair runs the kernel instance
// <kAnyDtype, void>, which picks the fold per part from the op's payload.  The 8-bit floats
// narrow under the FP16_OVFL mode bit, which also changes how binary16 overflows, so that
// instance sets the bit for exactly the parts that need it.
constexpr int kAnyDtype = -1;

// Not inlined: one function per dtype keeps the any-dtype kernel a small caller of eight
// mid-sized functions (as one flat function its compilation took minutes).
template <int DT>
__device__ __attribute__((noinline)) void run_part_any_compute(const pccl_op_payload *pl, const pccl_op_payload *more, long lo, long count) {
  switch (pl->compute_) {
    case PCCL_SUM: run_reduce_part<DT, OpSum, true>(pl, more, lo, count); break;
    case PCCL_PROD: run_reduce_part<DT, OpProd, true>(pl, more, lo, count); break;
    case PCCL_MIN: run_reduce_part<DT, OpMin, true>(pl, more, lo, count); break;
    default: run_reduce_part<DT, OpMax, true>(pl, more, lo, count); break;
  }
}

__device__ __forceinline__ void run_part_any(const pccl_op_payload *pl, const pccl_op_payload *more, long lo, long count) {
  if (pl->n_in_ == 1) {
    run_copy_part(pl, more, lo, count);
    return;
  }
  const int dt = pl->chunks_[0].dtype_;
  if (dt == PCCL_F8E4M3 || dt == PCCL_F8E5M2) {
    asm volatile("s_setreg_imm32_b32 hwreg(HW_REG_MODE, 23, 1), 1\n\ts_nop 1" ::: "memory");
  } else {
    asm volatile("s_setreg_imm32_b32 hwreg(HW_REG_MODE, 23, 1), 0\n\ts_nop 1" ::: "memory");
  }
  switch (dt) {
    case PCCL_F32: run_part_any_compute<PCCL_F32>(pl, more, lo, count); break;
    case PCCL_I32: run_part_any_compute<PCCL_I32>(pl, more, lo, count); break;
    case PCCL_BF16: run_part_any_compute<PCCL_BF16>(pl, more, lo, count); break;
    case PCCL_F16: run_part_any_compute<PCCL_F16>(pl, more, lo, count); break;
    case PCCL_F8E4M3: run_part_any_compute<PCCL_F8E4M3>(pl, more, lo, count); break;
    case PCCL_F8E5M2: run_part_any_compute<PCCL_F8E5M2>(pl, more, lo, count); break;
    case PCCL_F64: run_part_any_compute<PCCL_F64>(pl, more, lo, count); break;
    default: run_part_any_compute<PCCL_U32>(pl, more, lo, count); break;
  }
}

// ---- a whole chain in one pass -----------------------------------------------------
// For chains in which every op after the first reads the previous op's output 0 as one of at most two
// inputs (a ring step: what the neighbour produced, plus the local chunk; or a plain copy of it) and nothing
// else of the chain's outputs is read inside the chain: the value a lane has just stored is the value the
// next op would load, so it stays in registers.  Packs are cut so that the first op's output 0 is 16-byte
// aligned; the other operands are read and written at whatever element-aligned address that gives them.
// Per pack a lane loads the first op's inputs and every later op's other input up front (they depend on
// nothing), then folds and stores op after op.  The 14-op chain of a ring all-reduce over 8 resident
// ranks reads 8 packs and writes 14 instead of reading 21 and writing 14, with no store -> load round
// trip between the steps.  Bit for bit what the ops give one after the other: each step rounds to the
// element type exactly where the store would.
template <class D, class Op>
__device__ __forceinline__ u32x4 fold_two(const u32x4 &a, const u32x4 &b) {
  const u32x4 v[2] = {a, b};
  return fold_pack<D, Op, 2>(v);
}

// What the pass needs to know of one op of the chain.  The host keeps a table of these rows beside the
// payloads (and moves the addresses with them on a rebind); a part stages its chain's rows in LDS with
// one load per lane.  Walking the chain op by op through the payloads costs three dependent loads per
// op (next op, its payload, the operand address): 2 us per op on an idle device, more under load, and
// that was all the time the pass took.
struct ForwardStep {
  unsigned long long other;   // the input that is not handed on (ops after the first with two inputs), else 0
  unsigned long long out[2];  // outputs
  int n_out;
  int fed;                    // which input the handed-on value is (two-input ops after the first)
};
static_assert(sizeof(ForwardStep) == 32, "two 16-byte loads per row");

// The signal ops a data op carries (graph_queue.hip, fuse_signals): values are the ops' own, the run's
// signal base is added by the kernel.
struct SignalFuse {
  unsigned long long wait_word;    // 0: none
  unsigned long long notify_word;  // 0: none
  unsigned int wait_value, notify_value;  // | kSignalPerPart: the signal is a word per part, part p's is word p
};
constexpr unsigned int kSignalPerPart = 1u << 31;
constexpr unsigned int kSignalValue = 0xffffu;
static_assert(sizeof(SignalFuse) == 24, "three 8-byte words per row");

__device__ __forceinline__ unsigned long long uniform64(unsigned long long v) {  // the same in every lane: into scalar registers
  const unsigned int lo = __builtin_amdgcn_readfirstlane((unsigned int)v), hi = __builtin_amdgcn_readfirstlane((unsigned int)(v >> 32));
  return ((unsigned long long)hi << 32) | lo;
}

// kBatch: packs a lane carries through the chain at a time (4: 16 KiB per workgroup and stream);
// kAhead: ops whose other input is requested ahead of the value reaching them.
template <class D, class Op, int kBatch = 4, int kAhead = 4>
__device__ __forceinline__ void run_chain_forward(const GraphControl &g, const pccl_op_payload *hp, int n_steps, int first_row, long lo, long count) {
  typedef typename D::elem_t E;
  constexpr int kEpp = 16 / D::kElemBytes;
  __shared__ __attribute__((aligned(16))) ForwardStep s_step[kMaxForwardSteps];
  // (the first three operands' addresses together with the input count: which of them is output 0 depends
  // on the count, and a load that waits for the count would be one more round trip in front of the data:
  // ring all-reduce 8 x 8 / 16 / 32 MiB as a wide launch 23.4 / 49 / 86.7 -> 22.5 / 46 / 84.8 us)
  const int head_n_in = hp->n_in_;
  const char *head_in0 = (const char *)hp->chunks_[0].addr_, *head_a1 = (const char *)hp->chunks_[1].addr_, *head_a2 = (const char *)hp->chunks_[2].addr_;
  if (threadIdx.x < 2u * (unsigned)n_steps)  // two lanes per row
    ((u32x4 *)s_step)[threadIdx.x] = ((const u32x4 *)(g.chain_table + first_row))[threadIdx.x];
  __syncthreads();
  // the elements before output 0's first 16-byte boundary are left to the edge code below
  const unsigned long long out0 = (unsigned long long)(head_n_in == 2 ? head_a2 : head_a1) + (unsigned long long)lo * D::kElemBytes;
  long peel = (long)((16 - (out0 & 15)) & 15) / D::kElemBytes;
  if (peel > count) peel = count;
  const long n_packs = (count - peel) / kEpp;
  const size_t body = (size_t)(lo + peel) * D::kElemBytes;  // byte offset of the first pack from every operand's base
  for (long base = 0; base < n_packs; base += (long)kBlock * kBatch) {
    const size_t chunk = body + (size_t)base * 16;  // uniform
    const long left = n_packs - base;               // packs from here on; the lane's pack u exists if threadIdx.x + u * kBlock < left
    unsigned int off[kBatch];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const long q = (long)threadIdx.x + (long)u * kBlock;
      off[u] = (unsigned int)((q < left ? q : left - 1) * 16);  // a lane without pack u re-reads the last pack and stores nothing for it
    }
    // The loads of a chain depend on nothing the chain computes, so they go out well ahead of the
    // value: the first op's inputs and the other input of the ops among the next kAhead that have one,
    // together (up to 24 packs per lane in flight), then fold and store op after op, then the next
    // kAhead.  Within a group no load stands behind a store in the wavefront's queue (its wait counter
    // treats completion as in order, and a write-through store's acknowledgement takes microseconds).
    // Bytes in flight per round trip count for more than round trips: 4 packs x 4 ops ahead against
    // 2 x 8 (one group for a ring chunk's six folds instead of two): 4096-op schedule 89 -> 82 us, ring
    // all-reduce 8 x 8 MiB 42 -> 34 us, 8 x 32 MiB 110 -> 97 us (8 x 1 MiB 16.5 -> 18.4 us: its 8 KiB
    // parts are half a block); 3 x 6: 98 / 33 / 100 us.
    u32x4 cur[kBatch], in1[kBatch];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      cur[u] = load_pack<D, true, kMemCoherent>(head_in0 + chunk, off[u]);
      if (head_n_in == 2) in1[u] = load_pack<D, true, kMemCoherent>(head_a1 + chunk, off[u]);
    }
    for (int s0 = 0; s0 < n_steps; s0 += kAhead) {
      u32x4 other[kAhead][kBatch];
#pragma unroll
      for (int i = 0; i < kAhead; ++i) {
        const int s = s0 + i;
        if (s == 0 || s >= n_steps) continue;
        const unsigned long long from = uniform64(s_step[s].other);
        if (from == 0ull) continue;
#pragma unroll
        for (int u = 0; u < kBatch; ++u) other[i][u] = load_pack<D, true, kMemCoherent>((const char *)from + chunk, off[u]);
      }
      if (s0 == 0 && head_n_in == 2) {
#pragma unroll
        for (int u = 0; u < kBatch; ++u) cur[u] = fold_two<D, Op>(cur[u], in1[u]);
      }
#pragma unroll
      for (int i = 0; i < kAhead; ++i) {
        const int s = s0 + i;
        if (s >= n_steps) continue;
        if (s > 0 && uniform64(s_step[s].other) != 0ull) {
          const int fed = __builtin_amdgcn_readfirstlane(s_step[s].fed);
#pragma unroll
          for (int u = 0; u < kBatch; ++u) cur[u] = fed == 0 ? fold_two<D, Op>(cur[u], other[i][u]) : fold_two<D, Op>(other[i][u], cur[u]);
        }
        const int n_out = __builtin_amdgcn_readfirstlane(s_step[s].n_out);
        for (int j = 0; j < n_out; ++j) {
          char *to = (char *)uniform64(s_step[s].out[j]) + chunk;
#pragma unroll
          for (int u = 0; u < kBatch; ++u)
            if ((long)threadIdx.x + (long)u * kBlock < left) store_pack<D, true, kMemCoherent>(to, off[u], cur[u]);
        }
      }
    }
  }
  // the elements before the first pack and behind the last one (fewer than two packs' worth): one per
  // lane of the last wavefront, again with every load ahead of the first store
  if (threadIdx.x >= kBlock - kWave) {
    const long tail_begin = peel + n_packs * kEpp, n_edge = peel + (count - tail_begin);
    const long e = (long)threadIdx.x - (kBlock - kWave);
    if (e < n_edge) {
      const long i = lo + (e < peel ? e : tail_begin + (e - peel));
      E cur = load_elem<E, kMemCoherent>((const E *)head_in0 + i), second = cur;
      if (head_n_in == 2) second = load_elem<E, kMemCoherent>((const E *)head_a1 + i);
      E other[kMaxForwardSteps];
#pragma unroll
      for (int s = 1; s < kMaxForwardSteps; ++s) {
        other[s] = cur;
        if (s >= n_steps) continue;
        const unsigned long long from = uniform64(s_step[s].other);
        if (from != 0ull) other[s] = load_elem<E, kMemCoherent>((const E *)from + i);
      }
      if (head_n_in == 2) {
        const E x[2] = {cur, second};
        cur = D::template elem<Op, 2>(x);
      }
#pragma unroll
      for (int s = 0; s < kMaxForwardSteps; ++s) {
        if (s >= n_steps) continue;
        if (s > 0 && uniform64(s_step[s].other) != 0ull) {
          const int fed = __builtin_amdgcn_readfirstlane(s_step[s].fed);
          E x[2];
          x[fed] = cur;
          x[1 - fed] = other[s];
          cur = D::template elem<Op, 2>(x);
        }
        const int n_out = __builtin_amdgcn_readfirstlane(s_step[s].n_out);
        for (int j = 0; j < n_out; ++j) store_elem<E, kMemCoherent>((E *)uniform64(s_step[s].out[j]) + i, cur);
      }
    }
  }
}

#define AGENT __HIP_MEMORY_SCOPE_AGENT

// Trace record of a queue entry (entry t of queue q is record t * kQueues + q), times in ticks
// of the constant 100 MHz clock: who ran what, when the ticket was drawn, when the op's
// dependencies were met, when the part was complete.
constexpr int kTraceWords = 4;
constexpr int kTraceWhat = 0;     // op uid | part << 32 | workgroup << 52
constexpr int kTraceClaimed = 1;
constexpr int kTraceReady = 2;
constexpr int kTraceDone = 3;

// Polls `ready` until it holds.  Gives up (and raises the abort word, so that every workgroup
// leaves) once the wait has lasted spin_limit microseconds by the device's constant 100 MHz clock, or
// when another workgroup has given up.  A time, not a number of polls: how fast a poll returns
// depends on what else the device is doing.  (The clock is looked at every 64 polls.)
template <class Ready>
__device__ __forceinline__ bool bounded_wait(unsigned int *abort_flag, unsigned int spin_limit, Ready ready) {
  unsigned int spins = 0;
  unsigned long long since = 0;  // 0: the clock has not been looked at yet
  while (!ready()) {
    __builtin_amdgcn_s_sleep(1);
    if ((++spins & 63u) == 0) {
      const unsigned long long now = wall_clock64() | 1ull;
      if (since == 0) since = now;
      if (now - since >= (unsigned long long)spin_limit * 100ull ||
          __hip_atomic_load(abort_flag, __ATOMIC_RELAXED, AGENT) != 0) {
        __hip_atomic_store(abort_flag, 1u, __ATOMIC_RELAXED, AGENT);
        return false;
      }
    }
  }
  return true;
}

// Thread 0, after a part of op `h` is complete: count it; the op's last part re-arms
// the op's counters for the next run and releases its successors.
// `draw_ticket` requests the workgroup's next ticket; it is called exactly once, at the point
// where its round trip costs least: right behind the first counting atomic whose result this
// function has to wait for (the two then travel together), or, when nothing is counted
// (single-part op), after the successors have been told, so that their release is not held up
// behind the ticket (memory operations of a wavefront return in order).
// `notify` stores the signal word of the NOTIFY the op carries (a successor list can end in kSuccNotify).
template <class DrawTicket, class Notify>
__device__ __forceinline__ void finish_part(const GraphControl &g, pccl_operation_layout_header *h,
                                            const OpFacts &op, int uid, int part, unsigned int *done_ops, int chain_ops,
                                            DrawTicket draw_ticket, Notify notify) {
  const int parts = op.parts;
  // successors that need only this part of the op (they come first in the successor list):
  // part `part` of each is told right away
  const int n_part_next = op.part_nexts();
  if (n_part_next) {
    const int *first_entry = g.succ_part_base + op.succ_start;
    for (int s = 0; s < n_part_next; ++s)
      __hip_atomic_fetch_add(&g.part_arrivals[(size_t)(first_entry[s] + part) << g.part_shift], 1u, __ATOMIC_RELAXED, AGENT);
  }
  int counted = parts;  // what remaining_executors_ counts: parts, or groups of parts
  bool drawn = false;
  if (parts > kGroupThreshold) {
    const int group = part % kPartGroups;
    unsigned int *word = &g.groups[g.group_base[uid] + group].value;
    const unsigned int before = __hip_atomic_fetch_sub(word, 1u, __ATOMIC_RELAXED, AGENT);
    draw_ticket();
    drawn = true;
    if (before != 1u) return;
    // this group is done: re-arm it (parts p < parts with p % kPartGroups == group)
    __hip_atomic_store(word, (unsigned int)((parts - group + kPartGroups - 1) / kPartGroups), __ATOMIC_RELAXED, AGENT);
    counted = kPartGroups;
  }
  int old = 1;
  if (counted > 1) {
    old = __hip_atomic_fetch_sub(&h->remaining_executors_, 1, __ATOMIC_RELAXED, AGENT);
    if (!drawn) draw_ticket();
    drawn = true;
  }
  if (old != 1) return;
  if (counted > 1) __hip_atomic_store(&h->remaining_executors_, counted, __ATOMIC_RELAXED, AGENT);
  // The op is complete.  Its own arrivals word goes back to zero for the next run (every
  // dependency of this op has arrived, or it could not have run), and it arrives at each
  // successor: one add on the successor's arrivals word, whose result nobody waits for.  The
  // workgroups that already hold parts of a successor poll that word until it equals the
  // successor's pre_dependencies_ -- not the header, whose line the counting atomics of this
  // and neighbouring ops need (with 1024 pollers on a header line a hand-over between two
  // 32 MiB ops took 6 us longer), and without an atomic whose result decides who announces
  // (that round trip was a third of the latency between two dependent ops).
  if (op.pre_dependencies() > op.part_preds())
    __hip_atomic_store(&g.ready[uid].value, 0u, __ATOMIC_RELAXED, AGENT);
  const int n_next = op.num_next_ops();
  const int *next = g.succ + op.succ_start;
  for (int s = n_part_next; s < n_next; ++s) {
    const int to = next[s];
    if (to == kSuccNotify) notify(uid);  // (every part waited for its stores: the op has a successor)
    else __hip_atomic_fetch_add(&g.ready[to].value, 1u, __ATOMIC_RELAXED, AGENT);
  }
  // (an op that heads a chain stands for all the chain's ops: they ran behind it, part by part)
  *done_ops += (unsigned int)chain_ops;  // (the workgroup reports its count when it leaves)
  if (!drawn) draw_ticket();
}

// The kernel's body.  FORWARD: with the code that runs a chain in one pass (run_chain_forward).  That
// code needs 80 registers more than the rest, and compiled into the one kernel it cost graphs
// without such chains 3 % (14 ops of 32 MiB: 197 -> 203 us), so it is an instance of its own.
template <int DT, class Op, bool FORWARD>
__device__ __forceinline__ void drain_body(const GraphControl &g) {
  __shared__ unsigned long long s_entry;
  __shared__ i32x4 s_chain;  // the claimed op's kChainWords words
  __shared__ i32x4 s_facts;  // ... its part count, successor list and dependency counts (OpFacts)
  __shared__ long s_count;   // ... and its element count
  __shared__ int s_go;
  __shared__ int s_quit;  // with s_go == 0: the workgroup leaves because the run was given up, not because the queues are empty
  __shared__ int s_last;
  __shared__ unsigned int s_done;  // ops this workgroup has completed (thread 0 only)
  if (threadIdx.x == 0) s_done = 0;
  if constexpr (DT != kAnyDtype) Dtype<DT>::wave_init();
  HotWord *hot = g.hot;
  unsigned int *abort_flag = &hot[kHotAbort].value;
  const unsigned int spin_limit = g.spin_limit;
  const int home = blockIdx.x % kQueues;
  // Entries without tickets: workgroup b takes entries b, b + W, b + 2 W, ... of the global order (W
  // workgroups; entry b / kQueues + k * W / kQueues of its home queue) and leaves when its home queue
  // has no more.  No ticket is drawn, and no workgroup goes round the eight queues at the end to find
  // each of them empty (eight returning atomics, one after the other: 14.9 -> 11 us for a graph of one
  // 64 KiB op).  The host asks for it (mode word) when the entries are few per workgroup and none of
  // them waits for another entry of the graph: an entry then never waits for a workgroup that the
  // dispatcher has not started yet.
  // The mode word sits behind the queue lengths in memory, not in the kernel arguments: a rebind can
  // change the number of entries (see GraphControl::queue_count).  Thread 0 reads it before its first
  // claim, together with the entry that would be its own (a load from inside the queue's room even
  // where it is not used), and keeps it as a bit of `exhausted`.
  constexpr unsigned int kOwnEntry = 1u << 31, kAllQueues = (1u << kQueues) - 1u;
  // Thread 0 keeps the queue lengths in LDS: it needs one at every claim, and a scalar load that has
  // dropped out of the cache costs a trip to the L2 behind the data traffic (0.6 us per part measured).
  __shared__ int s_queue_count[kQueues + 1];  // [kQueues]: the workgroup's next entry on its home queue (entries without tickets)
  const int own_stride = (int)((gridDim.x + kQueues - 1) / kQueues);

  // Loop shape matters: thread 0's bookkeeping for the part just finished and its
  // claim of the next entry sit in ONE conditional block per iteration, and the
  // loop exit is a scalar branch (readfirstlane).  With two thread-0 blocks (one
  // before the back edge, one after it) the compiler threads the jump between
  // them, the back edge becomes divergent, and the other lanes of thread 0's
  // wavefront run ahead into the next barrier while thread 0 is parked.
  pccl_operation_layout_header *h = nullptr;
  const PayloadSlot *slot = nullptr;
  int cur_uid = 0, cur_part = 0;  // the entry being executed (uniform)
  OpFacts cur_op = {1, 0, 0};     // ... and its op's facts (uniform)
  int cur_chain_ops = 1;          // ... and how many ops it stands for: the chain it heads, or itself
  unsigned long long cur_entry = 0;         // the entry itself, flags included (thread 0 only)
  unsigned long long *cur_trace = nullptr;  // its trace record (thread 0 only)
  unsigned int exhausted = 0;  // bit q: queue q has no entries left (thread 0 only)
  // Signal values are offset by (run number << 16).  The run number lives on the device (not
  // in the kernel arguments) so that a launch recorded into a HIP graph uses a fresh one on
  // every replay; it is read at the first signal op, always before the last workgroup out of
  // this run bumps it.
  unsigned int signal_base = 0;
  bool have_signal_base = false;
  for (;;) {
    if (threadIdx.x == 0) {
      // The part executed in the previous iteration is complete (barrier below): every
      // wavefront waited for its write-through stores before that barrier, so the data is
      // at the point of coherence and relaxed device-scope atomics are enough to hand it
      // over; no L2 write-back / invalidate is involved.
      // The next ticket is requested while the finished part is being counted, so that the
      // two round trips overlap instead of following each other (see finish_part).
      int first_q = -1, first_t = 0;
      unsigned int aborted = 0;
      unsigned long long own_e = 0;
      // the workgroup's next entry without a ticket: its place on the home queue, requested at once if there is one
      auto next_own = [&] {
        const int t = s_queue_count[kQueues];
        s_queue_count[kQueues] = t + own_stride;
        if (t < s_queue_count[home]) own_e = g.queue_entries[home][t];
        return t;
      };
      auto draw_ticket = [&] {
        if (!h) {
          // The workgroup's first claim.  A ticket of its home queue is requested before the mode word
          // and the queue lengths are there (there are no more workgroups than entries at creation, so
          // the home queue has an entry for it); without tickets it goes unused, and the queue heads it
          // moved are set back with all the others when the run ends.
          const int ticket = __hip_atomic_fetch_add(g.queue_head[home], 1, __ATOMIC_RELAXED, AGENT);
          const int mode = g.queue_count[kQueues];
          own_e = g.queue_entries[home][blockIdx.x / kQueues];
#pragma unroll
          for (int q = 0; q < kQueues; ++q) s_queue_count[q] = g.queue_count[q];
          first_q = home;
          if (mode) {
            exhausted = kOwnEntry | (kAllQueues & ~(1u << home));  // (only the home queue is this workgroup's business)
            first_t = (int)(blockIdx.x / kQueues);
            s_queue_count[kQueues] = first_t + own_stride;
          } else {
            first_t = ticket;
            aborted = __hip_atomic_load(abort_flag, __ATOMIC_RELAXED, AGENT);
          }
          return;
        }
        if (exhausted & kOwnEntry) {
          first_q = home;
          first_t = next_own();
          aborted = __hip_atomic_load(abort_flag, __ATOMIC_RELAXED, AGENT);
          return;
        }
        for (int i = 0; i < kQueues && first_q < 0; ++i) {
          const int q = (home + i) % kQueues;
          if (!(exhausted & (1u << q)) && s_queue_count[q] > 0) first_q = q;
        }
        if (first_q >= 0) first_t = __hip_atomic_fetch_add(g.queue_head[first_q], 1, __ATOMIC_RELAXED, AGENT);
        aborted = __hip_atomic_load(abort_flag, __ATOMIC_RELAXED, AGENT);
      };
      auto base_of_run = [&] {
        if (!have_signal_base) {
          signal_base = __hip_atomic_load(&hot[kHotRun].value, __ATOMIC_RELAXED, AGENT) << 16;
          have_signal_base = true;
        }
        return signal_base;
      };
      // (graphs whose data ops carry signal ops run the plain instance: this one has no registers to spare)
      auto notify = [&](int uid) {
        if constexpr (!FORWARD) {
          const SignalFuse *f = &g.fuse[uid];
          __hip_atomic_store((unsigned int *)f->notify_word, base_of_run() + (f->notify_value & kSignalValue), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        }
      };
      if (h) {
        if (cur_trace) cur_trace[kTraceDone] = wall_clock64();
        // the NOTIFY of a word per part that the op carries: this part's word (its stores were waited for)
        if (!FORWARD && (cur_entry & kEntryNotifiesPart)) {
          const SignalFuse *f = &g.fuse[cur_uid];
          __hip_atomic_store((unsigned int *)f->notify_word + cur_part, base_of_run() + (f->notify_value & kSignalValue),
                             __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        }
        // (a part that is not counted goes the way of a single-part op without successors: nothing but the next ticket)
        OpFacts counted = cur_op;
        const bool uncounted = (cur_entry & kEntryUncounted) != 0;
        if (uncounted) counted.parts = 1;
        finish_part(g, h, counted, cur_uid, cur_part, &s_done, uncounted ? 0 : cur_chain_ops, draw_ticket, notify);
      } else {
        draw_ticket();
      }
      int go = 0;
      unsigned long long e = 0;
      i32x4 chain_words = {-1, 1, 0, 0};
      i32x4 op_facts = {1, 0, 0, 0};
      long op_count = 0;
      size_t entry_index = 0;  // of e in the global order
      int quit = 0;
      // claim entries until one needs the whole workgroup (COPY / REDUCE); signal ops
      // (NOTIFY / GET_NOTIFIED) are carried out right here by thread 0
      for (;;) {
        go = 0;
        if (aborted) {
          quit = 1;
          break;
        }
        for (int i = 0; i < kQueues && !go; ++i) {
          const int q = (home + i) % kQueues;
          if (exhausted & (1u << q)) continue;
          const int n = s_queue_count[q];
          int t = n;
          if (q == first_q) {  // the ticket requested above
            t = first_t;
            first_q = -1;
          } else if (exhausted & kOwnEntry) {  // (behind a signal op, which thread 0 has carried out itself)
            t = next_own();
          } else if (n > 0) {
            t = __hip_atomic_fetch_add(g.queue_head[q], 1, __ATOMIC_RELAXED, AGENT);
          }
          if (t < n) {
            // Only lane 0 is here, so "the first lane's value" is the value: with the index
            // uniform, this load and those of the op's slot and header below are scalar loads,
            // which do not queue behind the vector memory traffic of the parts in flight on
            // this compute unit.  What they read is constant during a run.
            const int qs = __builtin_amdgcn_readfirstlane(q), ts = __builtin_amdgcn_readfirstlane(t);
            e = (exhausted & kOwnEntry) ? own_e : g.queue_entries[qs][ts];
            entry_index = (size_t)ts * kQueues + qs;
            go = 1;
            if (g.trace) {
              cur_trace = g.trace + entry_index * kTraceWords;
              cur_trace[kTraceWhat] = (e & ~kEntryFlags) | ((unsigned long long)blockIdx.x << 52);
              cur_trace[kTraceClaimed] = wall_clock64();
            }
            if (t == 0 && q == 0) __hip_atomic_store(&hot[kHotCompleted].value, 0u, __ATOMIC_RELAXED, AGENT);
          } else {
            // A ticket came back without an entry.  The workgroup's own queue: go on to the next one, where
            // the neighbouring XCD's workgroups may be behind (under load every other XCD of this part is a
            // few per cent slower).  That one too: leave.  The queues run out at about the same time (entries
            // are dealt round-robin), and asking all eight, a returning atomic each, one after the other, kept
            // the last workgroups of every run for seven round trips with nothing to find.  Every queue keeps
            // the workgroups it is home to until it is empty, so no entry is left behind; with fewer
            // workgroups than queues some queue is nobody's home and every queue is asked.
            exhausted |= (q != home && gridDim.x >= (unsigned int)kQueues) ? kAllQueues : (1u << q);
          }
        }
        if (!go) break;
        const int uid = __builtin_amdgcn_readfirstlane((int)(e & 0xffffffffu));
        pccl_operation_layout_header *hc = &g.headers[uid];
        const PayloadSlot *sc = (const PayloadSlot *)(g.slots + (size_t)uid * kPayloadStride);
        // wait until every dependency of the op has arrived (none: nothing ever writes the
        // word); pre_dependencies_ in the header is the count to reach and stays constant.
        // The count, the first look at the arrivals and the primitive go out together.
        // Dependencies met part by part arrive on the entry's own word instead; the entry is
        // that word's only reader and clears it for the next run.
        const unsigned int w12 = *word12(hc);
        const unsigned int arrived = __hip_atomic_load(&g.ready[uid].value, __ATOMIC_RELAXED, AGENT);
        unsigned int *part_word = g.part_arrivals ? g.part_arrivals + ((size_t)(g.entry_base[uid] + (int)((e & ~kEntryFlags) >> 32)) << g.part_shift) : nullptr;
        const unsigned int part_arrived = part_word ? __hip_atomic_load(part_word, __ATOMIC_RELAXED, AGENT) : 0u;
        const int prim = sc->payload.primitive_;
        const unsigned int part_preds = sc->payload.part_preds_;
        // ... and with them what every wavefront needs to cut the part (part count and successor list from
        // the far end of the slot, the element count), handed over through LDS: read after the barrier
        // they were one more memory round trip in front of every part
        op_facts = i32x4{sc->parts, sc->succ_start, (int)*(const unsigned int *)&sc->payload.pre_dependencies_, 0};
        op_count = sc->payload.chunks_[0].num_elems_;
        if (e & kEntryChainHead) chain_words = *(const i32x4 *)(g.chain + kChainWords * uid);
        else chain_words = i32x4{-1, 1, 0, 0};
        const unsigned int n_pred = (w12 & 0xffu) - part_preds;  // whole-op dependencies
        if (n_pred != 0 && arrived != n_pred &&
            !bounded_wait(abort_flag, spin_limit, [&] {
              return __hip_atomic_load(&g.ready[uid].value, __ATOMIC_RELAXED, AGENT) == n_pred;
            })) {
          go = 0;
          quit = 1;
          break;
        }
        if (part_preds != 0) {
          if (part_arrived != part_preds &&
              !bounded_wait(abort_flag, spin_limit, [&] {
                return __hip_atomic_load(part_word, __ATOMIC_RELAXED, AGENT) == part_preds;
              })) {
            go = 0;
            quit = 1;
            break;
          }
          __hip_atomic_store(part_word, 0u, __ATOMIC_RELAXED, AGENT);
        }
        // the GET_NOTIFIED the op carries: every part polls the word before it starts
        if (!FORWARD && (e & kEntryWaitsSignal)) {
          const SignalFuse *f = &g.fuse[uid];
          const unsigned int value = f->wait_value;
          // (a word per part: this part's)
          unsigned int *word = (unsigned int *)f->wait_word + ((value & kSignalPerPart) ? (int)((e & ~kEntryFlags) >> 32) : 0);
          const unsigned int want = base_of_run() + (value & kSignalValue);
          if ((int)(__hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) - want) < 0 &&
              !bounded_wait(abort_flag, spin_limit, [&] {
                return (int)(__hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) - want) >= 0;
              })) {
            go = 0;
            quit = 1;
            break;
          }
        }
        if (cur_trace) cur_trace[kTraceReady] = wall_clock64();
        if (prim != PCCL_NOTIFY && prim != PCCL_GET_NOTIFIED) break;
        unsigned int *sig = (unsigned int *)sc->payload.chunks_[0].addr_;
        const unsigned int want = base_of_run() + (unsigned int)sc->payload.chunks_[0].num_elems_;
        // (a signal of a word per part that no data op carries: all of its words)
        const int n_words = (int)sc->payload.chunks_[1].num_elems_;
        bool gave_up = false;
        for (int w = 0; w < n_words && !gave_up; ++w) {
          if (prim == PCCL_NOTIFY) {
            // everything this op depends on is already at the point of coherence
            __hip_atomic_store(sig + w, want, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
          } else if (!bounded_wait(abort_flag, spin_limit, [&] {
                       return (int)(__hip_atomic_load(sig + w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) - want) >= 0;
                     })) {
            gave_up = true;
          }
        }
        if (gave_up) {
          go = 0;
          quit = 1;
          break;
        }
        if (cur_trace) cur_trace[kTraceDone] = wall_clock64();
        if (!(e & kEntryUncounted)) finish_part(g, hc, OpFacts::of(sc), uid, 0, &s_done, 1, [] {}, notify);
        aborted = __hip_atomic_load(abort_flag, __ATOMIC_RELAXED, AGENT);
      }
      s_entry = e;
      cur_entry = e;
      s_go = go;
      s_quit = quit;
      s_chain = chain_words;
      s_facts = op_facts;
      s_count = op_count;
    }
    __syncthreads();
    if (!__builtin_amdgcn_readfirstlane(s_go)) break;
    const int uid = __builtin_amdgcn_readfirstlane((int)(s_entry & 0xffffffffu));
    const int part = __builtin_amdgcn_readfirstlane((int)((s_entry & ~kEntryFlags) >> 32));
    const bool notifies_part = __builtin_amdgcn_readfirstlane((int)((s_entry & kEntryNotifiesPart) >> 53)) != 0;  // (its stores are waited for)
    cur_uid = uid;
    cur_part = part;
    h = &g.headers[uid];
    slot = (const PayloadSlot *)(g.slots + (size_t)uid * kPayloadStride);
    const pccl_op_payload *pl = &slot->payload;
    cur_op.parts = __builtin_amdgcn_readfirstlane(s_facts[0]);
    cur_op.succ_start = __builtin_amdgcn_readfirstlane(s_facts[1]);
    cur_op.counts = (unsigned int)__builtin_amdgcn_readfirstlane(s_facts[2]);
    const int chain_next = __builtin_amdgcn_readfirstlane(s_chain[kChainNext]);
    cur_chain_ops = __builtin_amdgcn_readfirstlane(s_chain[kChainLength]);
    const long count = (long)uniform64((unsigned long long)s_count);
    const long per = part_elems(count, cur_op.parts);
    const long lo = (long)part * per;
    long n = count - lo;
    if (n > per) n = per;
    if (n > 0) {
      bool forwarded = false;
      if constexpr (FORWARD && DT != kAnyDtype) {
        if (chain_next >= 0 && __builtin_amdgcn_readfirstlane(s_chain[kChainForward])) {
          run_chain_forward<Dtype<DT>, Op>(g, pl, cur_chain_ops, __builtin_amdgcn_readfirstlane(s_chain[kChainRow]), lo, n);
          forwarded = true;
        }
      }
      if (!forwarded) {
        // The op, then the ops chained behind it, same part: every wavefront has waited for its own
        // stores (run_part ends that way), the barrier makes that true of the whole workgroup, and the
        // next op's loads read past the L2 like every load here.  The chain index is uniform.
        // (One call site for both: a second inlined copy of run_part cost the kernel its registers.)
        const pccl_op_payload *step = pl;
        for (int next = chain_next;;) {
          // a COPY of this op's output 0 right behind it: this op stores the copy's outputs too (run_part_nin)
          const pccl_op_payload *more = nullptr;
          if (next >= 0 && g.chain[kChainWords * next + kChainForward] == kChainFolded) {
            more = &((const PayloadSlot *)(g.slots + (size_t)next * kPayloadStride))->payload;
            next = g.chain[kChainWords * next + kChainNext];
          }
          if constexpr (DT == kAnyDtype) run_part_any(step, more, lo, n);
          else run_part<DT, Op>(step, more, lo, n);
          if (next < 0) break;
          settle_stores();
          __syncthreads();
          step = &((const PayloadSlot *)(g.slots + (size_t)next * kPayloadStride))->payload;
          next = g.chain[kChainWords * next + kChainNext];
        }
      }
    }
    // Every store of this part has reached the point of coherence before thread 0 hands the part
    // over at the top of the next iteration: each wavefront waits for its own write-through stores,
    // the barrier makes that true of the workgroup.  Where nobody is told (the op, or the chain's
    // last op, has no successor in the graph) nobody reads the data before the kernel has ended,
    // and the wait is left out: one memory round trip less for the last ops of a graph.
    // The barrier also keeps s_entry / s_go from being rewritten while still being read.
    if (cur_op.num_next_ops() > 0 || (notifies_part && !FORWARD)) settle_stores();
    __syncthreads();
  }

  // leave: the last workgroup out re-arms the graph for the next run.  One returning atomic per
  // workgroup carries three facts: "one more has left" (bits 0-15), "it left because the run was given
  // up" (counted in bits 16-31) and "it completed this many of the ops that are counted" (high word), so
  // the last one out knows whether the run was given up, and what to report, without reading anything else.  No wait
  // stands before it: what the workgroup told others during the run (arrivals, counts put back for
  // the next run) has either been waited for where it mattered or only matters to the next launch.
  unsigned int total_done = 0;
  bool aborted = false;
  if (threadIdx.x == 0) {
    unsigned long long *exits = (unsigned long long *)&hot[kHotExit].value;  // (the word has a 256-byte line to itself)
    const unsigned int quit = s_quit ? kExitQuit : 0u;
    const unsigned long long before = __hip_atomic_fetch_add(exits, ((unsigned long long)s_done << 32) | (unsigned long long)(quit + 1u), __ATOMIC_RELAXED, AGENT);
    s_last = (((unsigned int)before & (kExitQuit - 1u)) == gridDim.x - 1);
    aborted = (((unsigned int)before + quit) >> 16) != 0;
    // (after a run that nobody gave up every op is complete, also those that are not counted: finish_part)
    total_done = aborted ? (unsigned int)(before >> 32) + s_done : g.n_ops;
  }
  __syncthreads();
  if (!__builtin_amdgcn_readfirstlane(s_last)) return;
  if (threadIdx.x == 0) {
    // after a run that was given up the per-op state is inconsistent: leave it for the host to restore
    if (!aborted)
      for (int q = 0; q < kQueues; ++q) __hip_atomic_store(g.queue_head[q], 0, __ATOMIC_RELAXED, AGENT);
    __hip_atomic_store(&hot[kHotCompleted].value, total_done, __ATOMIC_RELAXED, AGENT);
    __hip_atomic_store((unsigned long long *)&hot[kHotExit].value, 0ull, __ATOMIC_RELAXED, AGENT);
    __hip_atomic_fetch_add(&hot[kHotRun].value, 1u, __ATOMIC_RELAXED, AGENT);
  }
}

template <int DT, class Op>
__global__ void __launch_bounds__(kBlock) drain_graph_kernel(const GraphControl g) {  // by value: every field arrives through the kernarg segment
  drain_body<DT, Op, false>(g);
}

// (three wavefronts per SIMD like the plain instance: the allocator's own choice was two)
template <int DT, class Op>
__global__ void __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(3, 3))) drain_graph_forward_kernel(const GraphControl g) {
  drain_body<DT, Op, true>(g);
}

typedef void (*DrainKernel)(const GraphControl);

// ---- the wide launch ---------------------------------------------------------------------
// A graph none of whose queue entries waits for another entry (independent ops, chains: everything
// that depends on something runs behind it in the same workgroup) needs no queue at run time: which
// workgroup carries out which entry can be fixed by number, and nothing is handed from workgroup to
// workgroup.  Such a graph is cut into parts of one block (kWideTileBytes per stream) and launched
// in the shape of the direct kernels: one short-lived workgroup per entry, workgroup b takes entry b
// of the order the entries were dealt in, as many workgroups as entries.  The hardware dispatcher
// hands the next workgroup to whichever compute unit has room, so the faster XCDs carry out more
// entries, and no workgroup draws a ticket, looks at a dependency word or counts a part.  Against the
// persistent drain of the same graphs (ring all-reduce over 8 resident ranks, 112 ops in 8 chains):
// 8 x 1 MiB 16.7 -> 11 us, 8 x 8 MiB 31 -> 21 us, 8 x 32 MiB 93 -> 85 us, 8 x 64 MiB 225 -> 201 us.
// Nothing of the queue's state is written: no head moves, no part is counted, and the launch's end is
// the graph's completion.  The arena is the one the drain kernel would use (entries, payloads, chain
// words and table), so a rebind moves operands the same way.
constexpr long long kMaxWideEntries = 1ll << 20;  // workgroups of one wide launch (16 GiB of output in 16 KiB parts)
constexpr long kWideTileBytes = 16384;
constexpr long kWideSmallTileBytes = 8192;  // = kBlock lanes x 2 packs: the block of the SMALL instances  // = kBlock lanes x 4 packs: the block run_chain_forward carries through a chain

// SMALL: one-pass chains in blocks of kWideSmallTileBytes, two packs per lane with eight ops' inputs ahead,
// four wavefronts per SIMD: the better shape while the chains move little (ring all-reduce over 8 resident
// ranks x 1 / 8 / 16 MiB 11.4 / 22.9 / 46 -> 9.8 / 21.6 / 44.8 us), the worse one from 8 x 32 MiB (84.8 -> 89 us).
template <int DT, class Op, bool FORWARD, bool SMALL = false>
__device__ __forceinline__ void wide_body(const GraphControl &g) {
  if constexpr (DT != kAnyDtype) Dtype<DT>::wave_init();
  const unsigned int b = blockIdx.x;
  const WideEntry *we = &g.wide_entries[b];  // (uniform: scalar loads from here to the payload)
  const int uid = __builtin_amdgcn_readfirstlane(we->uid);
  const long n = (long)__builtin_amdgcn_readfirstlane(we->n);
  const long lo = (long)uniform64((unsigned long long)we->lo);
  const i32x4 chain = *(const i32x4 *)we->chain;
  const PayloadSlot *slot = (const PayloadSlot *)(g.slots + (size_t)uid * kPayloadStride);
  const pccl_op_payload *pl = &slot->payload;
  unsigned long long *trace = nullptr;
  if (threadIdx.x == 0 && g.trace && n > 0) {
    trace = g.trace + (size_t)b * kTraceWords;
    const unsigned long long now = wall_clock64();
    trace[kTraceWhat] = (unsigned long long)(unsigned int)uid | ((unsigned long long)(unsigned int)(lo / part_elems(pl->chunks_[0].num_elems_, slot->parts)) << 32) |
                        ((unsigned long long)(b & 0xfffu) << 52);
    trace[kTraceClaimed] = now;
    trace[kTraceReady] = now;
  }
  if (n > 0) {
    const int chain_next = __builtin_amdgcn_readfirstlane(chain[kChainNext]);
    bool forwarded = false;
    if constexpr (FORWARD && DT != kAnyDtype) {
      if (chain_next >= 0 && __builtin_amdgcn_readfirstlane(chain[kChainForward])) {
        run_chain_forward<Dtype<DT>, Op, SMALL ? 2 : 4, SMALL ? 8 : 4>(g, pl, __builtin_amdgcn_readfirstlane(chain[kChainLength]), __builtin_amdgcn_readfirstlane(chain[kChainRow]), lo, n);
        forwarded = true;
      }
    }
    if (!forwarded) {
      // the op, then the ops chained behind it, same part, through memory (as in drain_body)
      const pccl_op_payload *step = pl;
      for (int next = chain_next;;) {
        const pccl_op_payload *more = nullptr;
        if (next >= 0 && g.chain[kChainWords * next + kChainForward] == kChainFolded) {
          more = &((const PayloadSlot *)(g.slots + (size_t)next * kPayloadStride))->payload;
          next = g.chain[kChainWords * next + kChainNext];
        }
        if constexpr (DT == kAnyDtype) run_part_any(step, more, lo, n);
        else run_part<DT, Op>(step, more, lo, n);
        if (next < 0) break;
        settle_stores();
        __syncthreads();
        step = &((const PayloadSlot *)(g.slots + (size_t)next * kPayloadStride))->payload;
        next = g.chain[kChainWords * next + kChainNext];
      }
    }
  }
  // Nothing is counted on the way out: a workgroup that lives for a few microseconds would spend a
  // tenth of them waiting for a returning atomic (ring all-reduce 8 x 32 MiB: 85 -> 94 us with a count
  // per queue and an exit word).  The launch's end is the graph's completion; pccl_hip_graph_status
  // reports it in stream order, and *completed_operator on the device is not written by such a launch.
  if (trace) {
    __syncthreads();
    if (threadIdx.x == 0) trace[kTraceDone] = wall_clock64();
  }
}

template <int DT, class Op>
__global__ void __launch_bounds__(kBlock) wide_graph_kernel(const GraphControl g) {
  wide_body<DT, Op, false>(g);
}

template <int DT, class Op>
__global__ void __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(3, 3))) wide_graph_forward_kernel(const GraphControl g) {
  wide_body<DT, Op, true>(g);
}

template <int DT, class Op>
__global__ void __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(4, 4))) wide_graph_forward_small_kernel(const GraphControl g) {
  wide_body<DT, Op, true, true>(g);
}

// The instances, beside the drain kernel's in graph_queue_inst_<dtype>.hip / graph_queue_fwd_<dtype>.hip.
template <int DT>
DrainKernel wide_for_compute(int compute);
template <int DT>
DrainKernel wide_forward_for_compute(int compute);
template <int DT>
DrainKernel wide_forward_small_for_compute(int compute);
DrainKernel wide_for_any();

// The instances of one dtype; defined in graph_queue_inst_<dtype>.hip.
template <int DT>
DrainKernel drain_for_compute(int compute);
// ... and those with the one-pass chain code; defined in graph_queue_fwd_<dtype>.hip.
template <int DT>
DrainKernel drain_forward_for_compute(int compute);

// The instance for graphs whose REDUCE ops do not share one (dtype, compute) pair;
// defined in graph_queue_inst_any.hip.
DrainKernel drain_for_any();

#define PCCL_DEFINE_DRAIN_FOR_COMPUTE(DT)                        \
  template <>                                                    \
  DrainKernel drain_for_compute<DT>(int compute) {               \
    switch (compute) {                                           \
      case PCCL_SUM: return drain_graph_kernel<DT, OpSum>;       \
      case PCCL_PROD: return drain_graph_kernel<DT, OpProd>;     \
      case PCCL_MIN: return drain_graph_kernel<DT, OpMin>;       \
      default: return drain_graph_kernel<DT, OpMax>;             \
    }                                                            \
  }                                                              \
  template <>                                                    \
  DrainKernel wide_for_compute<DT>(int compute) {                \
    switch (compute) {                                           \
      case PCCL_SUM: return wide_graph_kernel<DT, OpSum>;        \
      case PCCL_PROD: return wide_graph_kernel<DT, OpProd>;      \
      case PCCL_MIN: return wide_graph_kernel<DT, OpMin>;        \
      default: return wide_graph_kernel<DT, OpMax>;              \
    }                                                            \
  }

#define PCCL_DEFINE_DRAIN_FORWARD_FOR_COMPUTE(DT)                        \
  template <>                                                    \
  DrainKernel drain_forward_for_compute<DT>(int compute) {               \
    switch (compute) {                                           \
      case PCCL_SUM: return drain_graph_forward_kernel<DT, OpSum>;       \
      case PCCL_PROD: return drain_graph_forward_kernel<DT, OpProd>;     \
      case PCCL_MIN: return drain_graph_forward_kernel<DT, OpMin>;       \
      default: return drain_graph_forward_kernel<DT, OpMax>;             \
    }                                                            \
  }                                                              \
  template <>                                                    \
  DrainKernel wide_forward_for_compute<DT>(int compute) {        \
    switch (compute) {                                           \
      case PCCL_SUM: return wide_graph_forward_kernel<DT, OpSum>;  \
      case PCCL_PROD: return wide_graph_forward_kernel<DT, OpProd>; \
      case PCCL_MIN: return wide_graph_forward_kernel<DT, OpMin>;  \
      default: return wide_graph_forward_kernel<DT, OpMax>;      \
    }                                                            \
  }                                                              \
  template <>                                                    \
  DrainKernel wide_forward_small_for_compute<DT>(int compute) {  \
    switch (compute) {                                           \
      case PCCL_SUM: return wide_graph_forward_small_kernel<DT, OpSum>;  \
      case PCCL_PROD: return wide_graph_forward_small_kernel<DT, OpProd>; \
      case PCCL_MIN: return wide_graph_forward_small_kernel<DT, OpMin>;  \
      default: return wide_graph_forward_small_kernel<DT, OpMax>;  \
    }                                                            \
  }

}  // namespace pccl_queue
