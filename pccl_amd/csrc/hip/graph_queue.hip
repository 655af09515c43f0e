// graph_queue.hip -- the op-batching path: a DAG of COPY / REDUCE ops lives on
// the device in the reference's GraphBufferLayout (include/base/operator.h:31-38)
// and ONE persistent kernel drains it; no launch per op.
//
// Protocol (the reference declares the structs, operator.h:7-38, but no code
// reads or writes them, so the protocol is defined here):
//   * an op is split into required_executors_ parts of about tile_bytes of
//     output (built-in choice: sized per dependency level, see "parts" below);
//     a queue entry names (op_uid, part);
//   * the entries of all ops are laid out once, at graph creation, in a
//     topological order (dependency level; inside a level by where the ops'
//     predecessors stand, then op id, the ops taking turns with blocks of parts) and dealt
//     round-robin onto kQueues ready queues (GraphBufferLayout::ready_queues /
//     num_queues; RingBuffer::tail_ = number of entries).  Workgroup w serves
//     queue w % kQueues first -- workgroups are dispatched round-robin over the 8
//     XCDs, so the ticket counter of a queue is hammered from one XCD only -- and
//     moves on to the other queues when its own is exhausted;
//   * a workgroup claims an entry by taking a ticket from RingBuffer::head_,
//     reads the entry, and waits until the op's dependencies have arrived (its arrivals
//     word equals pre_dependencies_, which itself stays constant).  Every
//     dependency of a claimed entry lies earlier in the global order; each queue
//     keeps at least one workgroup until it is exhausted; hence the unfinished
//     claimed entry that comes first in the global order can always run, and the
//     drain cannot deadlock whatever the number of resident workgroups;
//   * the workgroup finishing the last part of an op adds one to the arrivals word of
//     each successor (an atomic whose result nobody waits for) and clears its own;
//   * where a successor is cut like the op and touches the same bytes part for part,
//     its part p waits only for the op's part p (classify_dependencies below): every
//     part of the op bumps the word of the successor's entry p when it is complete;
//   * an op that follows one op alone, which nothing else needs, queues no entries: the
//     workgroup that ran part p of the one goes on with part p of the other (plan_chains
//     below), and where the value can stay in registers the whole chain is one pass;
//   * a NOTIFY behind one data op alone, and a GET_NOTIFIED in front of one data op alone, queue no
//     entries either: the op's last part stores the one word, every part of the op polls the other
//     (fuse_signals below);
//   * when there are no more entries than workgroups, workgroup b simply takes entry b
//     (no tickets; the mode word beside the queue lengths says so);
//   * data moves between workgroups (possibly on different XCDs, whose L2s are not
//     coherent with each other) through device-coherent accesses: parts load and
//     store with sc1, wait for their stores, and only then touch the counters with
//     relaxed device-scope atomics.  An L2-wide write-back + invalidate per part
//     (what agent-scope release / acquire fences compile to) was measured to cost
//     about 100 us per part under load;
//   * hot-spot atomics are the throughput limit (about 30-60 ns each on one
//     address): an earlier form with one queue, a tail_ reservation and a slot
//     store/poll per entry spent 2 contended atomics per entry on two addresses;
//     this form spends one, spread over kQueues addresses;
//   * per-op mutable state is restored by the op's last part and the run's
//     last workgroup rewinds the ticket counters, so a finished graph is armed
//     for its next run;
//   * every wait is bounded: when a wait has lasted spin_limit microseconds the kernel
//     raises the abort flag, all workgroups leave, and the host reports
//     PCCL_ERR_GRAPH instead of hanging.
#include <algorithm>
#include <cmath>
#include <cstring>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "graph_chains_device.h"
#include "graph_queue_device.h"

using namespace pccl_dev;
using namespace pccl_queue;
using pccl_host::fail;

namespace {

DrainKernel drain_for(int dtype, int compute, bool forward, bool wide = false, bool wide_small = false) {
  switch (dtype) {
    case PCCL_F32: return forward ? (wide ? (wide_small ? wide_forward_small_for_compute<PCCL_F32>(compute) : wide_forward_for_compute<PCCL_F32>(compute)) : drain_forward_for_compute<PCCL_F32>(compute))
                              : (wide ? wide_for_compute<PCCL_F32>(compute) : drain_for_compute<PCCL_F32>(compute));
    case PCCL_I32: return forward ? (wide ? (wide_small ? wide_forward_small_for_compute<PCCL_I32>(compute) : wide_forward_for_compute<PCCL_I32>(compute)) : drain_forward_for_compute<PCCL_I32>(compute))
                              : (wide ? wide_for_compute<PCCL_I32>(compute) : drain_for_compute<PCCL_I32>(compute));
    case PCCL_BF16: return forward ? (wide ? (wide_small ? wide_forward_small_for_compute<PCCL_BF16>(compute) : wide_forward_for_compute<PCCL_BF16>(compute)) : drain_forward_for_compute<PCCL_BF16>(compute))
                              : (wide ? wide_for_compute<PCCL_BF16>(compute) : drain_for_compute<PCCL_BF16>(compute));
    case PCCL_F16: return forward ? (wide ? (wide_small ? wide_forward_small_for_compute<PCCL_F16>(compute) : wide_forward_for_compute<PCCL_F16>(compute)) : drain_forward_for_compute<PCCL_F16>(compute))
                              : (wide ? wide_for_compute<PCCL_F16>(compute) : drain_for_compute<PCCL_F16>(compute));
    case PCCL_F8E4M3: return forward ? (wide ? (wide_small ? wide_forward_small_for_compute<PCCL_F8E4M3>(compute) : wide_forward_for_compute<PCCL_F8E4M3>(compute)) : drain_forward_for_compute<PCCL_F8E4M3>(compute))
                              : (wide ? wide_for_compute<PCCL_F8E4M3>(compute) : drain_for_compute<PCCL_F8E4M3>(compute));
    case PCCL_F8E5M2: return forward ? (wide ? (wide_small ? wide_forward_small_for_compute<PCCL_F8E5M2>(compute) : wide_forward_for_compute<PCCL_F8E5M2>(compute)) : drain_forward_for_compute<PCCL_F8E5M2>(compute))
                              : (wide ? wide_for_compute<PCCL_F8E5M2>(compute) : drain_for_compute<PCCL_F8E5M2>(compute));
    case PCCL_F64: return forward ? (wide ? (wide_small ? wide_forward_small_for_compute<PCCL_F64>(compute) : wide_forward_for_compute<PCCL_F64>(compute)) : drain_forward_for_compute<PCCL_F64>(compute))
                              : (wide ? wide_for_compute<PCCL_F64>(compute) : drain_for_compute<PCCL_F64>(compute));
    default: return forward ? (wide ? (wide_small ? wide_forward_small_for_compute<PCCL_U32>(compute) : wide_forward_for_compute<PCCL_U32>(compute)) : drain_forward_for_compute<PCCL_U32>(compute))
                              : (wide ? wide_for_compute<PCCL_U32>(compute) : drain_for_compute<PCCL_U32>(compute));
  }
}

// ---- host side ----------------------------------------------------------------

size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// How long a wait inside the kernel may last for a graph created from now on: two seconds, or
// PCCL_HIP_SPIN_LIMIT_US (at least 64; read at every creation).  pccl_hip_graph_set_spin_limit changes
// it for one graph; pccl_hip_graph_run_static, which hands out no graph, only has this.
unsigned int default_spin_limit() {
  if (const char *env = getenv("PCCL_HIP_SPIN_LIMIT_US")) {
    const long v = atol(env);
    if (v > 0) return (unsigned int)std::min<long>(std::max<long>(v, 64), 0x7fffffffl);
  }
  return kDefaultSpinLimit;
}

int elem_bytes(int dtype) { return pccl_host::pccl_dtype_bytes(dtype); }

struct Graph {
  char *dev = nullptr;          // device arena; starts with GraphControl
  size_t arena_bytes = 0;
  unsigned long long *trace = nullptr;  // device trace records, if tracing was switched on
  bool trace_on = false;
  unsigned int spin_limit = kDefaultSpinLimit;
  std::vector<char> image;      // pristine host copy of the arena
  size_t payload_off = 0;       // arena offset of the payload array
  size_t chain_table_off = 0;   // ... and of the chain table, which follows it
  int n_ops = 0;
  int total_tiles = 0;          // queue entries
  int all_tiles = 0;            // parts of all ops (>= total_tiles: an op that runs behind another in a chain queues none)
  int n_wg = 0;
  int fixed_n_wg = 0;           // build_graph: launch this many workgroups instead of choosing
  DrainKernel fixed_kernel = nullptr;  // build_graph: ... and this kernel instance
  bool forward_capable = false; // the instance has the code that runs a chain in one pass
  int kernel_elem_bytes = 0;    // element size of the instance's dtype
  int device = 0;
  unsigned int runs = 0;        // launches so far; run r uses signal values (r << 16) + value
  DrainKernel kernel = nullptr;
  std::mutex mu;
  // what the arena was built from (graph_rebind may have to build it again)
  std::vector<pccl_op_desc> descs;   // deps point into deps_store
  std::vector<int> deps_store;
  long tile_bytes = 0;               // as passed to graph_create
  std::vector<int> parts;            // per op
  std::vector<int> topo;             // a topological order of the ops
  std::vector<unsigned char> part_edge;  // per dependency, in descs order: met part by part
  std::vector<unsigned char> part_eligible;  // per op: its dependencies may be met part by part
  // chains (plan_chains): what the arena was built with; graph_rebind compares
  std::vector<int> n_succ;                 // per op: ops that depend on it
  std::vector<unsigned char> order_touch;  // per op: takes part in a NOTIFY -> GET_NOTIFIED ordering edge
  std::vector<int> chain_words;            // kChainWords ints per op, as uploaded
  // signal ops carried by data ops (fuse_signals): what build_graph works on
  std::vector<pccl_op_desc> eff;           // descs with the dependency lists rewritten; deps point into eff_deps
  std::vector<int> eff_deps;
  std::vector<int> fused_into;             // per op: the data op that carries this signal op, or -1
  std::vector<int> wait_of, notify_of;     // per op: the GET_NOTIFIED / NOTIFY it carries, or -1
  std::vector<int> signal_cut;             // per op: K if it carries signals of a word per part (it is then cut into K parts), else 0
  std::vector<long> user_dep_to_eff;       // per dependency as the caller listed them: its place among eff's, or -1
  size_t fuse_table_off = 0;               // arena offset of the carried signals' table (behind the chain table)
  std::vector<int> fixed_parts;            // build_graph: cut the ops like this instead of choosing (a rebuild in place:
                                           // the arena's layout, and with it its size, follows from the part counts)
  // The wide launch (graph_queue_device.h: wide_body): one workgroup per entry instead of the persistent drain.
  bool want_wide = false;  // build_graph: cut for it, check that the graph allows it, take its kernel
  bool wide_ok = false;    // build_graph's finding: no queue entry waits for another entry or for a signal
  bool wide_slow = false;  // ... but a long chain goes through memory op by op, which the drain does better
  bool wide = false;       // the graph runs that way
  long long wide_plain_bytes = 0;  // build_graph's finding: bytes moved by entries that do not run a chain in one pass
  int wide_plain_streams = 0;      // ... and the most operands such an entry walks at once (a copy stored by its producer counted in)
  std::vector<long> wide_tile_of;  // build_graph with want_wide: bytes per part, op by op (empty: kWideTileBytes for all)
  unsigned wide_lds = 0;           // dynamic LDS of the wide launch (never touched: an occupancy cap like the direct kernels')
  bool wide_small = false;         // one-pass chains in 8 KiB blocks (the SMALL instances of wide_body)
  long long wide_chain_bytes = 0;  // build_graph's finding: bytes the ops of one-pass chains name
  // A wide launch of a few chains that are each one fold (graph_chains_device.h): the kernel, its
  // arguments (the table of the chains' operands is in the arena at chains_off), its grid and LDS cap.
  bool chains_launch = false;
  ChainsKernel chains_kernel = nullptr;
  ChainsLaunch chains_args = {};
  size_t chains_off = 0;
  unsigned chains_grid = 0, chains_lds = 0;
  int chains_mem = 0, chains_dtype = 0, chains_compute = 0;
  const Graph *fixed_chains = nullptr;  // build_graph: the launch must come out like this graph's (a rebuild in place)
  // A graph that runs as plain launches instead (see plan_launches): no arena, no drain kernel.
  bool as_launches = false;
  std::vector<pccl_op_desc> launches;  // in an order that respects the dependencies (deps unused)
};

// How a graph that runs as a wide launch is cut and capped, from the plan of its first build (G).
// Chains that run in one pass: parts of one block (kWideTileBytes).  Everything else walks its part
// 4 KiB after 4 KiB like a direct launch of several packs per lane, for which the direct kernels' rules
// hold: much traffic wants longer parts and few workgroups per compute unit (about 20 workgroups x
// streams).  Direct all-reduce over 8 resident ranks (eight folds 8 -> 8), 16 KiB parts uncapped
// against 32 KiB parts at two workgroups per compute unit: 8 x 8 MiB 24.3 / 29.4 us, 8 x 16 MiB 58.6 /
// 47.5, 8 x 32 MiB 92.7 / 87.8, 8 x 64 MiB 221 / 215 (through the persistent drain 31.8 / 53 / 90.3 / 222).
void wide_cut_of(const Graph *G, Graph *W) {
  const bool much = G->wide_plain_bytes >= (192ll << 20);
  const int n = (int)G->eff.size();
  W->wide_tile_of.assign(n, kWideTileBytes);
  W->wide_lds = 0;
  std::vector<char> one_pass(n, 0);  // op belongs to a chain that runs in one pass (its head says so)
  for (int h = 0; h < n; ++h) {
    const int *w = &G->chain_words[(size_t)kChainWords * h];
    if (w[kChainNext] < 0 || w[kChainForward] != 1 || w[kChainLength] <= 1) continue;
    for (int u = h, k = 0; u >= 0 && k < w[kChainLength]; u = G->chain_words[(size_t)kChainWords * u + kChainNext], ++k) one_pass[u] = 1;
  }
  // One-pass chains whose ops name less than 512 MiB in all: blocks of 8 KiB and the SMALL kernel instance
  // (wide_body).  Ring all-reduce over 8 ranks x 1 / 8 MiB (37 / 294 MB named) 11.4 / 22.9 -> 9.6 / 21.8 us;
  // x 16 MiB (587 MB) would gain too (46 -> 44.7 us), but the 4096-op schedule (764 MB in 288 short chains)
  // loses (64 -> 67.8 us) and 8 x 32 MiB as well (84.8 -> 89 us).
  W->wide_small = G->wide_chain_bytes > 0 && G->wide_chain_bytes < (512ll << 20);
  if (W->wide_small)
    for (int i = 0; i < n; ++i)
      if (one_pass[i]) W->wide_tile_of[i] = kWideSmallTileBytes;
  if (!much) return;
  for (int i = 0; i < n; ++i)
    if (!one_pass[i]) W->wide_tile_of[i] = 2 * kWideTileBytes;
  const int streams = std::max(1, G->wide_plain_streams);
  const int wgs = std::max(2, std::min(8, (20 + streams / 2) / streams));
  if (wgs < 3) W->wide_lds = std::min(65536u, (unsigned)(160 * 1024 / wgs) - 256u);  // (the kernel's registers allow three)
}

// ---- which dependencies can be met part by part -------------------------------
// B depends on A.  Part p of B needs only part p of A when both ops are cut alike (same
// number of parts, same bytes per part and in all) and every pair of operands through which
// they conflict (A writes what B reads or writes, or A reads what B writes) starts at the
// same address: then part p of either op touches the same bytes of that pair.  A pair that
// overlaps at different addresses makes some other part of A matter and keeps the dependency
// whole-op.  No conflicting pair at all (the caller orders two ops that share no bytes) is met
// part by part as well: what a dependency promises here is that B is complete only after A is,
// and that everything B's parts touch is as A and A's own predecessors left it; both hold
// (every part of B waits for a part of A, and the rule below looks at what can still be in
// flight behind A), and who reads a NOTIFY behind B still knows A complete.  PCCL_HIP_ORDER_EDGES=0
// keeps such dependencies whole-op.
enum Conflict { kNoConflict, kSameAddress, kOtherAddress };
constexpr long long kMaxPartWordEntries = 1ll << 22;

Conflict conflict_of(const pccl_op_desc &a, const pccl_op_desc &b, uintptr_t bytes) {
  bool any = false, other = false;
  auto pair = [&](const void *x, const void *y) {
    const uintptr_t p = (uintptr_t)x, q = (uintptr_t)y;
    if (p < q + bytes && q < p + bytes) {
      any = true;
      if (p != q) other = true;
    }
  };
  for (int j = 0; j < a.n_out; ++j) {
    for (int k = 0; k < b.n_in; ++k) pair(a.outs[j], b.ins[k]);
    for (int k = 0; k < b.n_out; ++k) pair(a.outs[j], b.outs[k]);
  }
  for (int j = 0; j < a.n_in; ++j)
    for (int k = 0; k < b.n_out; ++k) pair(a.ins[j], b.outs[k]);
  return other ? kOtherAddress : any ? kSameAddress : kNoConflict;
}

// Flags per dependency (ops in index order, dependencies in list order).  behind[b] lists the
// ops that may still be running when a part of b starts: its part-by-part predecessors and
// theirs.  Whole-op semantics promise b that ALL its ancestors are complete, so b must not
// conflict with any op of behind[b] at differing addresses either; when it would, or when the
// list grows long, the dependency stays whole-op (which also empties what lies behind it).
// `eligible` (optional, per op): 0 keeps every dependency OF that op whole-op whatever the rule
// would allow (build_graph: graphs with too many entries for a part-arrival word each).
// Parts of one op that stand together in the order of the entries before the next op of the
// same dependency level takes its turn (PCCL_HIP_ORDER_BLOCK; 0 = all of them, i.e. op after
// op).  With op after op the workgroups in flight cover two or three large ops at a time; in
// blocks they work on every op of the level at once, each through a narrow window.  Measured on
// 14 32 MiB ring steps (7 reductions 2 -> 2, 7 copies; 256 parts each): op after op 208-210 us,
// blocks of 8 .. 64 parts 197-198 us, blocks of 128 214 us.  Most of that gain is the L2: each copy
// there reads the buffer a reduction reads too, and in blocks the two run side by side; with copies
// that read buffers of their own it is 212 -> 209 us.  Ring and direct all-reduces over 8 ranks x
// 1 .. 64 MiB and the 4096-op schedule (at most 3 parts per op) are unchanged within 1 %.
// Whether a graph that may run as a wide launch (wide_body) does: whenever it may.  Chains that run in
// one pass gain at every size measured (ring all-reduce over 8 resident ranks x 1 / 8 / 32 / 64 MiB:
// 16.4 / 31 / 93 / 227 us through the persistent drain, 11.9 / 23.4 / 87 / 196 us wide), and so do graphs
// of single ops and of chains through memory, cut as wide_cut_of says (one 64 KiB op 9.7 -> 6.5 us, the
// 4096-op schedule 77 -> 68 us, direct all-reduce 8 x 1 / 8 / 16 / 32 / 64 MiB 12.9 / 32 / 53 / 90.5 / 223 ->
// 9.9 / 24 / 46 / 89 / 218 us, 14 independent copies of 32 MiB 188 -> 156 us, 4096 independent 2 -> 1 ops
// of 64 KiB 73 -> 56 us, of 256 KiB 401 -> 403 us).
// PCCL_HIP_WIDE=0: never.
bool wide_launch_pays() {
  const char *env = getenv("PCCL_HIP_WIDE");
  return !(env && env[0] == '0');
}

int order_block() {
  int block = 32;
  if (const char *env = getenv("PCCL_HIP_ORDER_BLOCK")) block = atoi(env);
  return block > 0 ? block : 1 << 30;
}

// The last dependency level of a graph of several is the exception: its entries are the last ones
// drawn, and the run ends when the last of them does, so its ops go op after op with the ops whose
// parts move most bytes first, and the entries that a run ends with are its shortest.  One rank's 14
// ring steps of 32 MiB (last level: a reduction 2 -> 2 and a copy): 206.8 -> 205.7 us, through signal
// words 208.4 -> 207.2 us, as configured 197 -> 194-196 us.  PCCL_HIP_LAST_LEVEL=0: in blocks like the rest.
bool last_level_longest_first() {
  const char *env = getenv("PCCL_HIP_LAST_LEVEL");
  return !(env && env[0] == '0');
}

std::vector<unsigned char> classify_dependencies(const std::vector<pccl_op_desc> &ops, const std::vector<int> &parts,
                                                 const std::vector<int> &topo,
                                                 const std::vector<unsigned char> *eligible = nullptr) {
  constexpr size_t kMaxBehind = 32;
  const int n_ops = (int)ops.size();
  std::vector<size_t> dep_start(n_ops + 1, 0);
  for (int i = 0; i < n_ops; ++i) dep_start[i + 1] = dep_start[i] + (size_t)ops[i].n_deps;
  std::vector<unsigned char> flags(dep_start[n_ops], 0);
  if (const char *env = getenv("PCCL_HIP_PART_DEPS"))
    if (env[0] == '0') return flags;  // every dependency whole-op
  bool order_edges_by_part = true;
  if (const char *env = getenv("PCCL_HIP_ORDER_EDGES")) order_edges_by_part = env[0] != '0';
  std::vector<std::vector<int>> behind(n_ops);
  auto is_data = [&](const pccl_op_desc &o) { return o.primitive != PCCL_NOTIFY && o.primitive != PCCL_GET_NOTIFIED; };
  auto bytes_of = [&](const pccl_op_desc &o) { return (uintptr_t)o.count * (uintptr_t)elem_bytes(o.dtype); };
  for (int b : topo) {
    const pccl_op_desc &B = ops[b];
    if (!is_data(B) || parts[b] < 2 || (eligible && !(*eligible)[b])) continue;
    const uintptr_t bytes = bytes_of(B);
    const uintptr_t per = (uintptr_t)part_elems(B.count, parts[b]) * (uintptr_t)elem_bytes(B.dtype);
    for (int d = 0; d < B.n_deps; ++d) {
      const int a = B.deps[d];
      const pccl_op_desc &A = ops[a];
      if (!is_data(A) || parts[a] != parts[b] || bytes_of(A) != bytes ||
          (uintptr_t)part_elems(A.count, parts[a]) * (uintptr_t)elem_bytes(A.dtype) != per)
        continue;
      const Conflict how = conflict_of(A, B, bytes);
      if (how == kOtherAddress || (how == kNoConflict && !order_edges_by_part)) continue;
      bool ok = behind[a].size() + behind[b].size() + 1 <= kMaxBehind;
      for (size_t k = 0; ok && k < behind[a].size(); ++k)
        ok = conflict_of(ops[behind[a][k]], B, bytes) != kOtherAddress;
      if (!ok) continue;
      flags[dep_start[b] + d] = 1;
      auto add = [&](int x) {
        if (std::find(behind[b].begin(), behind[b].end(), x) == behind[b].end()) behind[b].push_back(x);
      };
      add(a);
      for (int x : behind[a]) add(x);
    }
  }
  return flags;
}

// Validates G->descs and builds the device arena and its host image from them.  On failure
// nothing is left allocated.  `run_number`: what the device's run word starts at.
// `reuse`: an arena of `reuse_bytes` to build into instead of allocating one (the arena's
// layout depends on the ops and their parts only, not on their addresses, so the arena of the
// same ops at other addresses fits exactly; a launch recorded by stream capture keeps
// pointing at it).
// ---- graphs that run faster as plain launches ------------------------------------------
// The queue is built for many ops: one op alone, however large, runs slower through it than as
// a direct launch (bf16 8 -> 1 at 256 MiB: 450 us against 354; one 64 KiB op: 13 us against 8),
// because every workgroup streams through a window of its own instead of the whole grid walking
// one window.  A caller of Engine::exeOp cannot choose the entry point, so graph_create may
// (tile_bytes == PCCL_HIP_TILE_AUTO).  Two rewrites first, both of which keep every byte written
// the same:
//   * a COPY whose only dependency is the op that wrote its input becomes more outputs of that
//     op (an all-reduce slice folded 8 -> 1 and then copied 1 -> 7 is one 8 -> 8 fold);
//   * independent ops of the same shape whose operands continue each other (slice d + 1 behind
//     slice d in every buffer) become one op.
// What is left runs as launches in dependency order if it is at most two ops, or at most four
// independent ops of at least 128 MiB of traffic each; anything else goes through the queue
// unchanged (a fused op can name 16 operands, the queue's payload 10).
bool plan_launches(const std::vector<pccl_op_desc> &ops, std::vector<pccl_op_desc> *plan) {
  const int n = (int)ops.size();
  if (n == 0) return false;
  if (const char *env = getenv("PCCL_HIP_PLAN_LAUNCHES"))
    if (env[0] == '0') return false;
  std::vector<pccl_op_desc> w(ops);
  std::vector<std::vector<int>> deps(n);
  std::vector<char> alive(n, 1);
  for (int i = 0; i < n; ++i) {
    const pccl_op_desc &o = w[i];
    if (o.primitive > PCCL_REDUCE || o.dtype >= PCCL_NUM_DTYPES || o.compute > PCCL_MAX || o.count < 0) return false;
    if (o.n_in < 1 || o.n_in > PCCL_MAX_INPUTS || o.n_out < 1 || o.n_out > PCCL_MAX_OUTPUTS) return false;
    if (o.primitive == PCCL_COPY && o.n_in != 1) return false;
    if (o.n_deps < 0 || (o.n_deps > 0 && !o.deps)) return false;
    for (int d = 0; d < o.n_deps; ++d) {
      if (o.deps[d] < 0 || o.deps[d] >= n || o.deps[d] == i) return false;
      deps[i].push_back(o.deps[d]);
    }
  }
  auto bytes_of = [&](const pccl_op_desc &o) { return (uintptr_t)o.count * (uintptr_t)elem_bytes(o.dtype); };
  // copies folded into the op that wrote their input
  for (bool changed = true; changed;) {
    changed = false;
    for (int b = 0; b < n; ++b) {
      if (!alive[b] || w[b].n_in != 1 || deps[b].size() != 1) continue;
      const int a = deps[b][0];
      pccl_op_desc &A = w[a], &B = w[b];
      if (!alive[a] || bytes_of(A) != bytes_of(B) || A.n_out + B.n_out > PCCL_MAX_OUTPUTS) continue;
      bool reads_a = false;
      for (int j = 0; j < A.n_out; ++j) reads_a = reads_a || A.outs[j] == B.ins[0];
      if (!reads_a) continue;
      // B's outputs must be new buffers to A: equal to none of A's operands and overlapping none
      bool clear = true;
      const uintptr_t len = bytes_of(A);
      auto overlaps = [&](const void *x, const void *y) {
        const uintptr_t p = (uintptr_t)x, q = (uintptr_t)y;
        return p < q + len && q < p + len;
      };
      for (int k = 0; k < B.n_out && clear; ++k) {
        for (int j = 0; j < A.n_in; ++j) clear = clear && !overlaps(B.outs[k], A.ins[j]);
        for (int j = 0; j < A.n_out; ++j) clear = clear && !overlaps(B.outs[k], A.outs[j]);
      }
      // nobody else may stand between them: an op that depends on A but not on B could read a buffer B
      // overwrites only if the graph already raced, so only direct successors of B are rewired
      if (!clear) continue;
      for (int k = 0; k < B.n_out; ++k) A.outs[A.n_out++] = B.outs[k];
      alive[b] = 0;
      for (int c = 0; c < n; ++c)
        for (int &d : deps[c])
          if (d == b) d = a;
      changed = true;
    }
  }
  // dependency order (ops are few when this matters; quadratic is fine up to the bound below)
  int n_alive = 0;
  for (int i = 0; i < n; ++i) n_alive += alive[i];
  if (n_alive > 64) return false;
  std::vector<int> order, indeg(n, 0);
  std::vector<char> has_succ(n, 0);
  for (int i = 0; i < n; ++i)
    if (alive[i]) {
      std::sort(deps[i].begin(), deps[i].end());
      deps[i].erase(std::unique(deps[i].begin(), deps[i].end()), deps[i].end());
      indeg[i] = (int)deps[i].size();
      for (int d : deps[i]) has_succ[d] = 1;
    }
  for (int round = 0; round < n_alive; ++round) {
    int pick = -1;
    for (int i = 0; i < n && pick < 0; ++i)
      if (alive[i] && indeg[i] == 0) pick = i;
    if (pick < 0) return false;  // a cycle: let graph_create report it
    order.push_back(pick);
    indeg[pick] = -1;
    for (int c = 0; c < n; ++c)
      if (alive[c] && indeg[c] > 0)
        for (int d : deps[c])
          if (d == pick) --indeg[c];
  }
  // independent ops of one shape whose operands continue each other become one op
  std::vector<pccl_op_desc> out;
  std::vector<char> free_standing;
  for (int i : order) {
    pccl_op_desc o = w[i];
    std::sort(o.outs, o.outs + o.n_out);  // every output gets the same bytes: their order is free
    const bool alone = deps[i].empty() && !has_succ[i];
    if (alone && !out.empty() && free_standing.back()) {
      pccl_op_desc &m = out.back();
      const uintptr_t step = bytes_of(m);
      bool cont = m.dtype == o.dtype && m.compute == o.compute && m.n_in == o.n_in && m.n_out == o.n_out &&
                  m.primitive == o.primitive;
      for (int k = 0; cont && k < o.n_in; ++k) cont = (uintptr_t)o.ins[k] == (uintptr_t)m.ins[k] + step;
      for (int k = 0; cont && k < o.n_out; ++k) cont = (uintptr_t)o.outs[k] == (uintptr_t)m.outs[k] + step;
      if (cont) {
        m.count += o.count;
        continue;
      }
    }
    o.n_deps = 0;
    o.deps = nullptr;
    out.push_back(o);
    free_standing.push_back(alone);
  }
  bool take = out.size() <= 2;
  if (!take && out.size() <= 4) {
    take = true;
    for (size_t k = 0; k < out.size(); ++k)
      take = take && free_standing[k] && (uintptr_t)(out[k].n_in + out[k].n_out) * bytes_of(out[k]) >= ((uintptr_t)128 << 20);
  }
  if (take) plan->swap(out);
  return take;
}

// ---- signal ops carried by data ops ------------------------------------------------
// A ring written the way ranks on different devices write it is, per step, GET_NOTIFIED -> data op ->
// NOTIFY, each a queue entry of its own with a hand-over through the arrival words between them (about
// 2.5 us each: a ring all-reduce over 8 resident ranks x 1 MiB took 106 us with signals against 18 us
// with plain dependencies).  Where the shape allows, the data op carries its neighbours instead:
//   * a NOTIFY that depends on one data op alone is stored by whoever completes that op (its last
//     part), and whatever depended on the NOTIFY depends on the data op;
//   * a GET_NOTIFIED that one data op alone depends on is polled by every part of that op before it
//     starts, and the op takes over the GET_NOTIFIED's own dependencies.
// A carried signal op queues no entry and is complete when its data op is.  One of each kind per data
// op; anything else stays an op of its own.  The plan depends on the ops' kinds and dependency lists
// only, never on addresses, so a rebind cannot change it.  PCCL_HIP_FUSE_SIGNALS=0 switches it off.
void fuse_signals(Graph *G) {
  const std::vector<pccl_op_desc> &user = G->descs;
  const int n = (int)user.size();
  G->fused_into.assign(n, -1);
  G->wait_of.assign(n, -1);
  G->notify_of.assign(n, -1);
  G->signal_cut.assign(n, 0);
  // A signal of a word per part (signal_parts = K >= 2) rides on a data op only if the op can be cut
  // into exactly K parts: it has no such signal yet, or one of the same K.
  auto words_of = [&](int v) { return user[v].signal_parts >= 2 ? (int)user[v].signal_parts : 0; };
  auto cut_allows = [&](int data_op, int v) {
    const int k = words_of(v);
    return k == 0 || G->signal_cut[data_op] == 0 || G->signal_cut[data_op] == k;
  };
  bool on = true;
  if (const char *env = getenv("PCCL_HIP_FUSE_SIGNALS")) on = env[0] != '0';
  std::vector<std::vector<int>> deps(n);
  bool sane = true;
  for (int i = 0; i < n && sane; ++i) {
    const pccl_op_desc &o = user[i];
    sane = o.n_deps >= 0 && (o.n_deps == 0 || o.deps) && o.primitive <= PCCL_GET_NOTIFIED;
    for (int d = 0; sane && d < o.n_deps; ++d) {
      sane = o.deps[d] >= 0 && o.deps[d] < n && o.deps[d] != i;
      if (sane) deps[i].push_back(o.deps[d]);
    }
  }
  auto is_data = [&](int i) { return user[i].primitive == PCCL_COPY || user[i].primitive == PCCL_REDUCE; };
  if (on && sane) {
    std::vector<int> n_succ(n, 0);
    for (int i = 0; i < n; ++i)
      for (int d : deps[i]) ++n_succ[d];
    // NOTIFYs first: what depended on a carried NOTIFY then depends on its data op
    std::vector<int> stands_for(n);
    for (int i = 0; i < n; ++i) stands_for[i] = i;
    for (int v = 0; v < n; ++v) {
      if (user[v].primitive != PCCL_NOTIFY || deps[v].size() != 1) continue;
      const int a = deps[v][0];
      if (!is_data(a) || G->notify_of[a] >= 0 || n_succ[a] - 1 + n_succ[v] > 255 || !cut_allows(a, v)) continue;
      if (words_of(v)) G->signal_cut[a] = words_of(v);
      G->notify_of[a] = v;
      G->fused_into[v] = a;
      stands_for[v] = a;
      n_succ[a] += n_succ[v] - 1;
      n_succ[v] = 0;
      deps[v].clear();
    }
    for (int i = 0; i < n; ++i) {
      for (int &d : deps[i]) d = stands_for[d];
      std::sort(deps[i].begin(), deps[i].end());
      deps[i].erase(std::unique(deps[i].begin(), deps[i].end()), deps[i].end());
    }
    // GET_NOTIFIEDs that one data op alone waits for
    std::vector<int> only_succ(n, -1), succ_count(n, 0);
    for (int i = 0; i < n; ++i)
      for (int d : deps[i]) {
        ++succ_count[d];
        only_succ[d] = i;
      }
    for (int v = 0; v < n; ++v) {
      if (user[v].primitive != PCCL_GET_NOTIFIED || succ_count[v] != 1) continue;
      const int b = only_succ[v];
      if (!is_data(b) || G->wait_of[b] >= 0 || !cut_allows(b, v)) continue;
      std::vector<int> merged;
      for (int d : deps[b])
        if (d != v) merged.push_back(d);
      merged.insert(merged.end(), deps[v].begin(), deps[v].end());
      std::sort(merged.begin(), merged.end());
      merged.erase(std::unique(merged.begin(), merged.end()), merged.end());
      if (merged.size() > 255) continue;
      if (words_of(v)) G->signal_cut[b] = words_of(v);
      G->wait_of[b] = v;
      G->fused_into[v] = b;
      deps[b].swap(merged);
      deps[v].clear();
    }
  }
  // the ops with the rewritten lists, and for every dependency the caller listed its place among them
  G->eff = user;
  G->eff_deps.clear();
  G->user_dep_to_eff.clear();
  if (!sane) return;  // (build_graph reports what is wrong with the lists, from the ops as they came)
  std::vector<size_t> start(n + 1, 0);
  for (int i = 0; i < n; ++i) {
    start[i] = G->eff_deps.size();
    G->eff_deps.insert(G->eff_deps.end(), deps[i].begin(), deps[i].end());
  }
  start[n] = G->eff_deps.size();
  for (int i = 0; i < n; ++i) {
    G->eff[i].n_deps = (int)(start[i + 1] - start[i]);
    G->eff[i].deps = G->eff[i].n_deps > 0 ? G->eff_deps.data() + start[i] : nullptr;
    for (int d = 0; d < user[i].n_deps; ++d) {
      long place = -1;
      if (G->fused_into[i] < 0 && G->fused_into[user[i].deps[d]] < 0)
        for (size_t k = start[i]; k < start[i + 1]; ++k)
          if (G->eff_deps[k] == user[i].deps[d]) place = (long)k;
      G->user_dep_to_eff.push_back(place);
    }
  }
}

// G->eff with the operands of `moved` (the same ops at other addresses)
std::vector<pccl_op_desc> effective_of(const Graph *G, const std::vector<pccl_op_desc> &moved) {
  std::vector<pccl_op_desc> e = G->eff;
  for (size_t i = 0; i < e.size(); ++i) {
    memcpy(e[i].ins, moved[i].ins, sizeof(e[i].ins));
    memcpy(e[i].outs, moved[i].outs, sizeof(e[i].outs));
  }
  return e;
}

// ---- chains -------------------------------------------------------------------
// B follows A in a chain when B depends on A alone, A is needed by B alone, both are cut alike and
// part p of B may start as soon as part p of A is complete (single-part ops: always; otherwise the
// part-by-part rule above).  Such a B gets no queue entries of its own: the workgroup that has run
// part p of A goes on with part p of B, and so on down the chain.  Nothing is claimed, counted,
// signalled or polled between the steps.  The chain's head carries the head's dependencies and the
// tail's successors; when its last part is done every op of the chain is complete.  (A ring
// all-reduce over ranks that live on one device is such chains, 14 ops long.)
// Two ways to run a chain's part (graph_queue_device.h): op after op through memory (a barrier
// between them), or, where every later op takes the previous op's output 0 as one of at most two
// inputs and reads nothing else that the chain writes, in one pass with the value handed on in
// registers ("forward").  (Packs are 16-byte aligned on the first op's output 0; the other operands
// may sit at any element-aligned address, as for any part in this kernel.)
// Returns kChainWords ints per op.
std::vector<int> plan_chains(const std::vector<pccl_op_desc> &ops, const std::vector<int> &parts,
                             const std::vector<unsigned char> &part_edge, const std::vector<int> &n_succ,
                             const std::vector<unsigned char> &order_touch, int forward_elem_bytes) {
  const int n_ops = (int)ops.size();
  std::vector<int> words((size_t)kChainWords * (size_t)std::max(n_ops, 1), 0);
  std::vector<int> next(n_ops, -1), prev(n_ops, -1);
  // forward_elem_bytes: element size of the kernel instance's dtype if it has the one-pass code, else 0.
  // A chain of copies may have another element size than the graph's REDUCE ops (a copy moves bytes
  // of its own dtype): such a chain goes through memory, where every op is run by its own rule.
  bool on = true, forward_on = forward_elem_bytes > 0, fold_copies = true;
  if (const char *env = getenv("PCCL_HIP_CHAINS")) on = env[0] != '0', forward_on = forward_on && (env[0] != '1' || env[1] != 'm');  // "1m": through memory only
  if (const char *env = getenv("PCCL_HIP_FOLD_COPIES")) fold_copies = env[0] != '0';
  auto is_data = [&](int i) { return ops[i].primitive != PCCL_NOTIFY && ops[i].primitive != PCCL_GET_NOTIFIED; };
  auto bytes_of = [&](int i) { return (uintptr_t)ops[i].count * (uintptr_t)elem_bytes(ops[i].dtype); };
  size_t at = 0;
  for (int i = 0; i < n_ops; ++i) {
    const size_t first_dep = at;
    at += (size_t)ops[i].n_deps;
    if (!on || ops[i].n_deps != 1 || order_touch[i] || !is_data(i)) continue;
    const int a = ops[i].deps[0];
    if (n_succ[a] != 1 || order_touch[a] || !is_data(a) || parts[a] != parts[i]) continue;
    if (ops[a].count != ops[i].count || elem_bytes(ops[a].dtype) != elem_bytes(ops[i].dtype)) continue;
    if (parts[i] > 1 && !part_edge[first_dep]) continue;
    next[a] = i;
    prev[i] = a;
  }
  for (int i = 0; i < n_ops; ++i) {
    words[(size_t)kChainWords * i + kChainNext] = next[i];
    words[(size_t)kChainWords * i + kChainLength] = 1;
  }
  int listed = 0;
  for (int h = 0; h < n_ops; ++h) {
    if (prev[h] >= 0 || next[h] < 0) continue;
    std::vector<int> steps;
    for (int u = h; u >= 0; u = next[u]) steps.push_back(u);
    words[(size_t)kChainWords * h + kChainLength] = (int)steps.size();
    // can the values be handed on in registers?
    bool forward = forward_on && (int)steps.size() <= kMaxForwardSteps && ops[h].n_in <= 2 &&
                   elem_bytes(ops[h].dtype) == forward_elem_bytes;
    for (int t : steps) forward = forward && ops[t].n_out <= 2;
    const uintptr_t len = bytes_of(h);
    std::vector<int> fed(steps.size(), 0);
    for (size_t s = 0; forward && s < steps.size(); ++s) {
      const pccl_op_desc &o = ops[steps[s]];
      if (s == 0 || !forward) continue;
      const void *handed = ops[steps[s - 1]].outs[0];
      if (o.n_in > 2) { forward = false; break; }
      int f = -1;
      for (int k = 0; k < o.n_in; ++k)
        if (o.ins[k] == handed && f < 0) f = k;
      if (f < 0) { forward = false; break; }
      fed[s] = f;
      // whatever else the op reads must be something the chain never writes
      for (int k = 0; k < o.n_in && forward; ++k) {
        if (k == f) continue;
        for (int t : steps)
          for (int j = 0; j < ops[t].n_out && forward; ++j) {
            const uintptr_t x = (uintptr_t)o.ins[k], y = (uintptr_t)ops[t].outs[j];
            if (x < y + len && y < x + len) forward = false;
          }
      }
    }
    // Two ops of the chain may write the same elements only at the same address (the later store then
    // comes from the same lane, behind the earlier one, or replaces it: fill_chain_table); ranges that
    // overlap at a shift would be written by different lanes in no particular order.
    for (size_t s1 = 0; forward && s1 < steps.size(); ++s1)
      for (size_t s2 = s1 + 1; forward && s2 < steps.size(); ++s2)
        for (int j = 0; j < ops[steps[s1]].n_out && forward; ++j)
          for (int k = 0; k < ops[steps[s2]].n_out && forward; ++k) {
            const uintptr_t x = (uintptr_t)ops[steps[s1]].outs[j], y = (uintptr_t)ops[steps[s2]].outs[k];
            if (x != y && x < y + len && y < x + len) forward = false;
          }
    // ... and the first op's inputs too (an in-place first op is fine: it reads before it writes, pack by pack)
    for (int k = 0; forward && k < ops[h].n_in; ++k)
      for (size_t s = 1; s < steps.size() && forward; ++s)
        for (int j = 0; j < ops[steps[s]].n_out && forward; ++j) {
          const uintptr_t x = (uintptr_t)ops[h].ins[k], y = (uintptr_t)ops[steps[s]].outs[j];
          if (x < y + len && y < x + len) forward = false;
        }
    if (forward) {
      words[(size_t)kChainWords * h + kChainForward] = 1;
      words[(size_t)kChainWords * h + kChainRow] = listed;  // first of its rows in the chain table (fill_chain_table)
      listed += (int)steps.size();
      for (size_t s = 1; s < steps.size(); ++s) words[(size_t)kChainWords * steps[s] + kChainForward] = fed[s];
    } else if (fold_copies) {
      // A chain that runs through memory: a COPY of the previous op's output 0 is not run at all, the
      // previous op stores the copy's outputs as further outputs of its own (what the fold of an
      // all-reduce slice followed by its broadcast copy is: 8 -> 1 then 1 -> 7 becomes 8 -> 8, with no
      // wait for the stores, barrier and read-back between the two).  The copy's outputs must be new
      // to the previous op: none of them may overlap one of its operands at another address (the lanes
      // of a part would write what other lanes still have to read), and together they fit one op.
      bool prev_folded = false;
      for (size_t s = 1; s < steps.size(); ++s) {
        const pccl_op_desc &A = ops[steps[s - 1]], &B = ops[steps[s]];
        bool fold = !prev_folded && B.n_in == 1 && B.ins[0] == A.outs[0] && A.n_out + B.n_out <= PCCL_MAX_OUTPUTS;
        for (int k = 0; fold && k < B.n_out; ++k) {
          const uintptr_t y = (uintptr_t)B.outs[k];
          for (int j = 0; fold && j < A.n_in; ++j) {
            const uintptr_t x = (uintptr_t)A.ins[j];
            if (x != y && x < y + len && y < x + len) fold = false;
          }
          for (int j = 0; fold && j < A.n_out; ++j) {
            const uintptr_t x = (uintptr_t)A.outs[j];
            if (x != y && x < y + len && y < x + len) fold = false;
          }
          for (int j = 0; fold && j < k; ++j) {
            const uintptr_t x = (uintptr_t)B.outs[j];
            if (x != y && x < y + len && y < x + len) fold = false;
          }
        }
        if (fold) words[(size_t)kChainWords * steps[s] + kChainForward] = kChainFolded;
        prev_folded = fold;
      }
    }
  }
  return words;
}

// The rows of GraphControl::chain_table, from the payloads as they stand in the host image: for
// every chain that runs in one pass, in op order of the heads, one row per op of the chain.
// An output that a later op of the same chain writes again at the same address is left out of its
// row: nothing can read the earlier value (the op's only successor is the next op of the chain, which
// gets the value in registers, and whatever else the chain reads is nothing the chain writes), and
// part p of the later op covers the same elements as part p of the earlier one.  In a ring
// all-reduce the partial sums that the reduce-scatter steps leave in the ranks' output buffers are
// such outputs, overwritten by the all-gather copies behind them: a chunk's chain then writes 8
// streams instead of 14.
void fill_chain_table(const std::vector<int> &words, int n_ops, const char *payloads, ForwardStep *rows) {
  std::vector<const pccl_op_payload *> steps;
  for (int h = 0; h < n_ops; ++h) {
    if (!words[(size_t)kChainWords * h + kChainForward] || words[(size_t)kChainWords * h + kChainLength] < 2) continue;
    ForwardStep *row = rows + words[(size_t)kChainWords * h + kChainRow];
    steps.clear();
    for (int u = h; u >= 0; u = words[(size_t)kChainWords * u + kChainNext])
      steps.push_back((const pccl_op_payload *)(payloads + kPayloadStride * (size_t)u));
    size_t at = 0;
    for (int u = h; u >= 0; u = words[(size_t)kChainWords * u + kChainNext], ++row, ++at) {
      const pccl_op_payload *pl = steps[at];
      const int fed = u == h ? 0 : words[(size_t)kChainWords * u + kChainForward];
      row->fed = fed;
      row->other = (u != h && pl->n_in_ == 2) ? (unsigned long long)(uintptr_t)pl->chunks_[1 - fed].addr_ : 0ull;
      row->n_out = 0;
      row->out[0] = row->out[1] = 0ull;
      for (int j = 0; j < pl->n_out_; ++j) {
        const void *addr = pl->chunks_[pl->n_in_ + j].addr_;
        bool written_again = false;
        for (size_t t = at + 1; t < steps.size() && !written_again; ++t)
          for (int k = 0; k < steps[t]->n_out_; ++k)
            if (steps[t]->chunks_[steps[t]->n_in_ + k].addr_ == addr) written_again = true;
        if (!written_again) row->out[row->n_out++] = (unsigned long long)(uintptr_t)addr;
      }
    }
  }
}

ChainsKernel chains_kernel_for(int dtype, int compute, int mem) {
  switch (dtype) {
    case PCCL_F32: return chains_for_compute<PCCL_F32>(compute, mem);
    case PCCL_I32: return chains_for_compute<PCCL_I32>(compute, mem);
    case PCCL_U32: return chains_for_compute<PCCL_U32>(compute, mem);
    case PCCL_F64: return chains_for_compute<PCCL_F64>(compute, mem);
    case PCCL_BF16: return chains_for_compute<PCCL_BF16>(compute, mem);
    case PCCL_F16: return chains_for_compute<PCCL_F16>(compute, mem);
    case PCCL_F8E4M3: return chains_for_compute<PCCL_F8E4M3>(compute, mem);
    default: return chains_for_compute<PCCL_F8E5M2>(compute, mem);
  }
}

// PCCL_HIP_CHAIN_LAUNCH=0: graphs that could run as graph_chains_kernel run as the table-driven wide launch;
// 2: every graph that fits that kernel runs as it, also where it is not the better choice (launch_chains_of).
int chain_launch_mode() {
  const char *env = getenv("PCCL_HIP_CHAIN_LAUNCH");
  return env && env[0] == '0' ? 0 : env && env[0] == '2' ? 2 : 1;
}

// The rows of a graph that runs as graph_chains_kernel (graph_chains_device.h), one per queued op in op
// order, from the ops as they stand and their chain words; false when the graph does not fit: more than
// kMaxLaunchChains queued ops, an op or chain that is not one fold with all surviving outputs holding its
// final value (a chain through memory other than a copy stored by its producer; an output of a one-pass
// chain that no later op overwrites although a later op still folds), more than kChainStreams inputs or
// outputs, a fold in another dtype or compute op than the graph's kernel, an op of another element size.
// *shape: kChainsFold if every chain folds at least two inputs and walks at least four streams, kChainsFanOut if
// every chain is a copy to at least three outputs, else 0: where the launch is the better choice (fan-out
// copies from 48 MiB in all, with the non-temporal stores a direct launch gives them).  Eight independent ops of
// 1 / 4 / 16 / 32 MiB per stream, table-driven wide launch against this one, us: copies 1 -> 1 7.2 / 15 /
// 44 / 81 against 7.8 / 17 / 53 / 103 and folds 2 -> 1 7.5 / 19 / 62 / 118 against 7.9 / 19 / 66 / 124, but
// 2 -> 2 8 / 23 / 80 / 183 against 8.5 / 23 / 83 / 167, 4 -> 1 9 / 30 / 106 / 209 against 9.8 / 26 / 101 / 192,
// 8 -> 1 15 / 56 / 222 / 440 against 14 / 53 / 189 / 368, 4 -> 4 15 / 47 / 205 / 401 against 14 / 45 / 178 / 340;
// fan-out copies with write-through stores lose a fifth around 256 MiB in all (1 -> 8 x 4 MiB 45 -> 55), with
// non-temporal stores 1 -> 3 8.4 / 26 / 101 / 206 against 9.3 / 23 / 77 / 149, 1 -> 4 9.6 / 30 / 132 / 267 against
// 10.5 / 28 / 95 / 188, 1 -> 8 14 / 45 / 240 / 510 against 14 / 45 / 166 / 355 (all-gather and broadcast over 8
// ranks x 8 / 32 / 128 MiB: 14 / 44 / 235 against 14 / 44 / 167 us).
// Which outputs survive depends on the operands' addresses, whether the graph fits does not, short of a
// rebind that changes the chains themselves.  The caller has made sure that no queued op waits for anything.
constexpr int kChainsFold = 1, kChainsFanOut = 2;
bool launch_chains_of(const std::vector<pccl_op_desc> &ops, const std::vector<int> &words, int dtype, int compute,
                      std::vector<LaunchChain> *rows, int *shape) {
  *shape = kChainsFold | kChainsFanOut;
  const int n = (int)ops.size();
  std::vector<char> member(n, 0);
  for (int i = 0; i < n; ++i) {
    const int next = words[(size_t)kChainWords * i + kChainNext];
    if (next >= 0) member[next] = 1;
  }
  rows->clear();
  for (int h = 0; h < n; ++h) {
    if (member[h]) continue;
    if ((int)rows->size() == kMaxLaunchChains) return false;
    std::vector<int> steps;
    for (int u = h; u >= 0; u = words[(size_t)kChainWords * u + kChainNext]) steps.push_back(u);
    const pccl_op_desc &head = ops[h];
    const long long bytes = (long long)head.count * elem_bytes(head.dtype);
    if (head.count <= 0 || bytes / 16 / kBlock >= (1ll << 31)) return false;
    LaunchChain c;
    memset(&c, 0, sizeof(c));
    c.uid = h;
    c.count = head.count;
    c.n_wg = (unsigned int)std::max<long long>(1, (bytes / 16 + kBlock - 1) / kBlock);
    bool ok = true;
    auto folds_like_the_kernel = [&](const pccl_op_desc &o) { return o.n_in == 1 || (o.dtype == dtype && o.compute == compute); };
    auto add_in = [&](const void *p) {
      if (c.n_in == kChainStreams) { ok = false; return; }
      c.in[c.n_in++] = (unsigned long long)(uintptr_t)p;
    };
    auto add_out = [&](const void *p) {
      if (c.n_out == kChainStreams) { ok = false; return; }
      c.out[c.n_out++] = (unsigned long long)(uintptr_t)p;
    };
    for (int u : steps) {
      const pccl_op_desc &o = ops[u];
      ok = ok && (o.primitive == PCCL_COPY || o.primitive == PCCL_REDUCE) && o.n_in >= 1 && o.n_in <= PCCL_MAX_INPUTS &&
           folds_like_the_kernel(o) && o.count == head.count && elem_bytes(o.dtype) == elem_bytes(dtype);
    }
    if (!ok) return false;
    c.n_head = head.n_in;
    for (int k = 0; k < head.n_in; ++k) add_in(head.ins[k]);
    const int forward = words[(size_t)kChainWords * h + kChainForward];
    if (steps.size() == 1) {
      for (int j = 0; j < head.n_out; ++j) add_out(head.outs[j]);
    } else if (forward == 1) {
      if (head.n_in > 2) ok = false;  // (the kernel folds a chain's head as 1 or 2 inputs: plan_chains hands on nothing else)
      size_t last_fold = 0;  // the last op that changes the value
      for (size_t t = 1; t < steps.size() && ok; ++t) {
        const pccl_op_desc &o = ops[steps[t]];
        if (o.n_in == 2) {
          const int fed = words[(size_t)kChainWords * steps[t] + kChainForward];
          if (fed == 1) c.fed |= 1u << c.n_in;
          add_in(o.ins[1 - fed]);
          last_fold = t;
        } else if (o.n_in != 1) {
          ok = false;
        }
      }
      for (size_t t = 0; t < steps.size() && ok; ++t)
        for (int j = 0; j < ops[steps[t]].n_out && ok; ++j) {
          const void *addr = ops[steps[t]].outs[j];
          bool written_again = false;  // (as in fill_chain_table)
          for (size_t later = t + 1; later < steps.size() && !written_again; ++later)
            for (int k = 0; k < ops[steps[later]].n_out; ++k) written_again = written_again || ops[steps[later]].outs[k] == addr;
          if (written_again) continue;
          if (t < last_fold) ok = false;  // an earlier value that stays in memory
          else add_out(addr);
        }
    } else if (steps.size() == 2 && words[(size_t)kChainWords * steps[1] + kChainForward] == kChainFolded) {
      for (int j = 0; j < head.n_out; ++j) add_out(head.outs[j]);
      for (int j = 0; j < ops[steps[1]].n_out; ++j) add_out(ops[steps[1]].outs[j]);
    } else {
      ok = false;
    }
    if (!ok || c.n_out < 1) return false;
    if (!(c.n_in >= 2 && c.n_in + c.n_out >= 4)) *shape &= ~kChainsFold;
    if (!(c.n_in == 1 && c.n_out >= 3)) *shape &= ~kChainsFanOut;
    rows->push_back(c);
  }
  return !rows->empty();
}

// plan_chains for a graph's ops, and in the length word of every op the signal ops it carries: a
// workgroup that completes the op counts those complete with it (such an op is in no chain, so the
// word would otherwise say 1).
std::vector<int> plan_chains_of(const Graph *G, const std::vector<pccl_op_desc> &ops, const std::vector<int> &parts,
                                const std::vector<unsigned char> &part_edge, int forward_elem_bytes) {
  std::vector<int> words = plan_chains(ops, parts, part_edge, G->n_succ, G->order_touch, forward_elem_bytes);
  for (size_t i = 0; i < ops.size(); ++i)
    words[(size_t)kChainWords * i + kChainLength] += (G->wait_of[i] >= 0) + (G->notify_of[i] >= 0);
  return words;
}

// Rows of GraphControl::fuse: per data op the signal word and value it waits for before every part and
// the ones it stores when its last part is complete (addresses as they stand in `ops`).
void fill_fuse_table(const Graph *G, const std::vector<pccl_op_desc> &ops, SignalFuse *rows) {
  for (size_t i = 0; i < ops.size(); ++i) {
    SignalFuse f = {0ull, 0ull, 0u, 0u};
    if (G->wait_of[i] >= 0) {
      const pccl_op_desc &w = ops[G->wait_of[i]];
      f.wait_word = (unsigned long long)(uintptr_t)w.ins[0];
      f.wait_value = (unsigned int)w.count | (w.signal_parts >= 2 ? kSignalPerPart : 0u);
    }
    if (G->notify_of[i] >= 0) {
      const pccl_op_desc &v = ops[G->notify_of[i]];
      f.notify_word = (unsigned long long)(uintptr_t)v.outs[0];
      f.notify_value = (unsigned int)v.count | (v.signal_parts >= 2 ? kSignalPerPart : 0u);
    }
    rows[i] = f;
  }
}

// What pccl_hip_reduce_copy would refuse about a planned launch's operands, found at creation time.
int check_launch(const pccl_op_desc &o) {
  const int es = elem_bytes(o.dtype);
  for (int k = 0; k < o.n_in + o.n_out; ++k) {
    const void *p = k < o.n_in ? o.ins[k] : o.outs[k - o.n_in];
    if (!p && o.count) return fail(PCCL_ERR_INVALID_ARG, "op %d: operand %d is null", o.op_uid, k);
    if ((uintptr_t)p % (uintptr_t)es) return fail(PCCL_ERR_MISALIGNED, "op %d: operand %d not %d-byte aligned", o.op_uid, k, es);
  }
  return PCCL_OK;
}

// `fixed`: build into this memory, which the caller owns and which is not allocated here (the
// arena must fit its capacity), and upload behind earlier work on its stream.
struct FixedArena {
  char *ptr;
  size_t capacity;
  hipStream_t stream;
};

int build_graph(Graph *G, unsigned int run_number, char *reuse = nullptr, size_t reuse_bytes = 0,
                const FixedArena *fixed = nullptr) {
  fuse_signals(G);  // from here on the ops are G->eff: the caller's, with signal ops folded into data ops where that is possible
  const pccl_op_desc *ops = G->eff.data();
  const int n_ops = (int)G->eff.size();
  auto carrier = [&](int i) { return G->fused_into[i] >= 0 ? G->fused_into[i] : i; };
  long tile_bytes = G->want_wide ? kWideTileBytes : G->tile_bytes;  // (a wide launch: every op in parts of one block)
  const bool default_tile = tile_bytes == 0;  // parts are then sized per dependency level, below
  if (!default_tile) tile_bytes = std::max<long>(tile_bytes, 1024);

  // ---- validate; one (dtype, compute) pair for all REDUCE ops --------------
  int g_dtype = -1, g_compute = -1;  // the (dtype, compute) pair of the REDUCE ops, if they share one
  bool mixed = false;
  std::vector<int> n_succ(n_ops, 0), n_pred(n_ops, 0), parts(n_ops, 1), signal_ops;
  size_t n_edges = 0;
  long long tiles = 0;
  std::vector<long> op_bytes(n_ops, 0);
  for (int i = 0; i < n_ops; ++i) {
    const pccl_op_desc &o = ops[i];
    if (o.op_uid != i) return fail(PCCL_ERR_GRAPH, "op %d: op_uid %d is not its index (uids are dense from 0)", i, o.op_uid);
    if (o.primitive > PCCL_GET_NOTIFIED)
      return fail(PCCL_ERR_UNSUPPORTED, "op %d: unknown primitive code %d", i, o.primitive);
    const bool is_signal = o.primitive == PCCL_NOTIFY || o.primitive == PCCL_GET_NOTIFIED;
    int es = 1;
    if (is_signal) {
      // NOTIFY: outs[0] is the signal word, GET_NOTIFIED: ins[0]; count is the value
      const bool notify = o.primitive == PCCL_NOTIFY;
      if (o.n_in != (notify ? 0 : 1) || o.n_out != (notify ? 1 : 0))
        return fail(PCCL_ERR_INVALID_ARG, "op %d: NOTIFY takes 0 inputs / 1 output, GET_NOTIFIED 1 input / 0 outputs", i);
      const void *sig = notify ? (const void *)o.outs[0] : o.ins[0];
      if (!sig) return fail(PCCL_ERR_INVALID_ARG, "op %d: signal address is null", i);
      if ((uintptr_t)sig % 4) return fail(PCCL_ERR_MISALIGNED, "op %d: signal address not 4-byte aligned", i);
      if (o.count < 0 || o.count > 0xffff)
        return fail(PCCL_ERR_INVALID_ARG, "op %d: signal value %ld outside [0, 65535]", i, o.count);
      if ((int)o.signal_parts > kMaxParts)
        return fail(PCCL_ERR_INVALID_ARG, "op %d: a signal of %d words (at most %d)", i, (int)o.signal_parts, kMaxParts);
      signal_ops.push_back(i);
    } else {
      if (o.dtype >= PCCL_NUM_DTYPES) return fail(PCCL_ERR_UNSUPPORTED, "op %d: unknown dtype code %d", i, o.dtype);
      if (o.compute > PCCL_MAX) return fail(PCCL_ERR_UNSUPPORTED, "op %d: unknown compute code %d", i, o.compute);
      if (o.n_in < 1 || o.n_in > PCCL_MAX_INPUTS || o.n_out < 1 || o.n_out > PCCL_MAX_OUTPUTS ||
          o.n_in + o.n_out > PCCL_MAX_OP_CHUNKS)
        return fail(PCCL_ERR_INVALID_ARG, "op %d: n_in %d / n_out %d (each 1..8, at most 10 operands in all)", i, o.n_in, o.n_out);
      if (o.primitive == PCCL_COPY && o.n_in != 1)
        return fail(PCCL_ERR_INVALID_ARG, "op %d: COPY takes exactly one input", i);
      if (o.count < 0) return fail(PCCL_ERR_INVALID_ARG, "op %d: count %ld < 0", i, o.count);
      if (o.signal_parts) return fail(PCCL_ERR_INVALID_ARG, "op %d: signal_parts belongs to NOTIFY / GET_NOTIFIED", i);
      es = elem_bytes(o.dtype);
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
        else if (g_dtype != o.dtype || g_compute != o.compute) mixed = true;
      }
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
    op_bytes[i] = is_signal ? 0 : o.count * es;
  }
  // An op that carries a NOTIFY has one more place in its successor list: kSuccNotify, behind the ops
  // (what completes the op walks that list anyway, and an op with a successor waits for its stores).
  // (a carried NOTIFY of a word per part has no place there: every part stores its own word)
  auto notifies_by_part = [&](int i) { return G->notify_of[i] >= 0 && ops[G->notify_of[i]].signal_parts >= 2; };
  for (int i = 0; i < n_ops; ++i)
    if (G->notify_of[i] >= 0 && !notifies_by_part(i)) {
      ++n_succ[i];
      ++n_edges;
    }
  for (int i = 0; i < n_ops; ++i)
    if (n_succ[i] > 255) return fail(PCCL_ERR_GRAPH, "op %d: %d successors exceed num_next_ops_ (unsigned char)", i, n_succ[i]);
  // copy-only graphs: the kernel instance of the first op's dtype (a chain of copies of that element
  // size can then run in one pass; nothing else depends on the choice)
  if (g_dtype < 0) {
    g_dtype = PCCL_BF16;
    g_compute = PCCL_SUM;
    for (int i = 0; i < n_ops; ++i)
      if (ops[i].primitive != PCCL_NOTIFY && ops[i].primitive != PCCL_GET_NOTIFIED) {
        g_dtype = ops[i].dtype;
        break;
      }
  }
  // launch width: as many workgroups as the chip holds of this kernel instance
  // (two instances per dtype and fold: with and without the code that runs a chain in one pass.  Which
  // of them runs is settled once the chains are known, below; the launch width must hold for both.  A
  // rebuild in place keeps the instance: launches that a stream capture has recorded carry it.)
  const bool wide = G->want_wide;
  const DrainKernel plain_kernel = mixed ? (wide ? wide_for_any() : drain_for_any()) : drain_for(g_dtype, g_compute, false, wide);
  // (the instance with the one-pass code has no registers to spare for carried signal ops: a graph with
  // such ops runs the plain one, its chains through memory)
  bool carries = false;
  for (int i = 0; i < n_ops; ++i) carries = carries || G->fused_into[i] >= 0;
  const DrainKernel forward_kernel = (mixed || carries) ? nullptr : drain_for(g_dtype, g_compute, true, wide, G->wide_small);
  const int forward_elem_bytes = (G->fixed_kernel ? G->forward_capable : (!mixed && !carries)) ? elem_bytes(g_dtype) : 0;
  int occ = 8;
  for (DrainKernel k : {plain_kernel, forward_kernel}) {
    if (!k) continue;
    int o = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&o, (const void *)k, kBlock, 0) != hipSuccess || o < 1) {
      (void)hipGetLastError();
      o = 4;
    }
    occ = std::min(occ, o);
  }
  // (fewer than kExitQuit: the exit word counts the workgroups that have left in 16 bits)
  const long long cap = std::min<long long>((long long)pccl_host::compute_units() * occ, (long long)kExitQuit - 1);
  // ---- acyclicity (Kahn) -----------------------------------------------------
  std::vector<int> succ_start(n_ops + 1, 0);
  for (int i = 0; i < n_ops; ++i) succ_start[i + 1] = succ_start[i] + n_succ[i];
  std::vector<int> succ(n_edges ? n_edges : 1, kSuccNotify), fill(n_ops, 0);  // (the places no op fills are the carried NOTIFYs')
  for (int i = 0; i < n_ops; ++i)
    for (int d = 0; d < ops[i].n_deps; ++d) {
      const int u = ops[i].deps[d];
      succ[succ_start[u] + fill[u]++] = i;
    }
  // A GET_NOTIFIED must not be claimed ahead of the NOTIFY that satisfies it (same signal
  // word, same value, same graph), or workgroups could fill up with waits nobody can end.
  // Such pairs are ordering edges: they count for levels and cycles, not for
  // pre_dependencies_ (the hand-over itself goes through the signal word).
  std::vector<std::vector<int>> order_succ(n_ops);
  std::vector<int> order_pred(n_ops, 0);
  {
    // NOTIFYs by signal word.  A GET_NOTIFIED(word, v) is satisfied by any NOTIFY(word, w >= v); it is
    // ordered behind the one with the smallest such w (the first that can release it).  When that
    // NOTIFY has another value than the GET asks for, the edge is only added if the GET is not
    // itself upstream of the NOTIFY (a wait that an outside party satisfies, followed by a later
    // notification on the same word, is a legitimate program, and the edge would close a cycle).
    std::unordered_map<const void *, std::vector<int>> notifies;
    for (int a : signal_ops)
      if (ops[a].primitive == PCCL_NOTIFY) notifies[ops[a].outs[0]].push_back(a);
    auto reaches = [&](int from, int to) {  // over dependency edges and the ordering edges so far
      std::vector<char> seen(n_ops, 0);
      std::vector<int> stack{from};
      seen[from] = 1;
      while (!stack.empty()) {
        const int u = stack.back();
        stack.pop_back();
        if (u == to) return true;
        for (int e = succ_start[u]; e < succ_start[u + 1]; ++e)
          if (succ[e] >= 0 && !seen[succ[e]]) { seen[succ[e]] = 1; stack.push_back(succ[e]); }
        for (int v : order_succ[u])
          if (!seen[v]) { seen[v] = 1; stack.push_back(v); }
      }
      return false;
    };
    for (int b : signal_ops) {
      if (ops[b].primitive != PCCL_GET_NOTIFIED) continue;
      auto it = notifies.find(ops[b].ins[0]);
      if (it == notifies.end()) continue;  // satisfied from outside the graph
      int best = -1;
      for (int a : it->second)
        if (ops[a].count >= ops[b].count && (best < 0 || ops[a].count < ops[best].count)) best = a;
      if (best < 0) continue;
      // (carried signal ops stand where their data ops stand)
      const int from = carrier(best), to = carrier(b);
      if (from == to) continue;
      if (ops[best].count != ops[b].count && reaches(to, from)) continue;
      if (std::find(order_succ[from].begin(), order_succ[from].end(), to) != order_succ[from].end()) continue;
      order_succ[from].push_back(to);
      ++order_pred[to];
    }
  }
  // level[i] = length of the longest dependency chain ending in op i
  std::vector<int> level(n_ops, 0);
  {
    std::vector<int> indeg(n_ops), stack;
    G->topo.clear();
    G->topo.reserve(n_ops);
    for (int i = 0; i < n_ops; ++i) {
      indeg[i] = n_pred[i] + order_pred[i];
      if (!indeg[i]) stack.push_back(i);
    }
    int seen = 0;
    auto relax = [&](int u, int v) {
      level[v] = std::max(level[v], level[u] + 1);
      if (--indeg[v] == 0) stack.push_back(v);
    };
    while (!stack.empty()) {
      const int u = stack.back();
      stack.pop_back();
      G->topo.push_back(u);
      ++seen;
      for (int e = succ_start[u]; e < succ_start[u + 1]; ++e)
        if (succ[e] >= 0) relax(u, succ[e]);
      for (int v : order_succ[u]) relax(u, v);
    }
    if (seen != n_ops) return fail(PCCL_ERR_GRAPH, "dependency graph has a cycle (%d of %d ops reachable)", seen, n_ops);
  }
  // ---- parts ------------------------------------------------------------------
  std::vector<int> parts_by_level;  // the built-in choice for ops outside chains
  // A given tile_bytes cuts every op into parts of that size.  The built-in choice works per
  // dependency level and grows with the bytes the level writes: part = 16 KiB x (level bytes /
  // 8 MiB)^(2/3), within 8 KiB .. 128 KiB (for the 768 workgroups an MI355X holds of this kernel;
  // scaled for another count), never more parts per op than workgroups.  That puts a level of 8 MiB
  // at 0.67 rounds of the resident workgroups, 32 MiB at about one round, 64 MiB at 1.33.  Measured
  // best part sizes it was fitted to (ring all-reduces over 8 virtual ranks of 1 / 8 / 32 / 64 MiB,
  // the 4096-op schedule, one rank's 14 ring steps of 32 MiB ordered by their buffer hazards):
  // levels of 8 MiB 16 KiB (12 KiB +10 %, 20 KiB +10 %), 18 MiB 32 KiB (16 KiB +29 %, 64 KiB +10 %),
  // 32 MiB 47 KiB, 64 MiB 64-76 KiB (14 ring steps: 96 KiB +8 %, 128 KiB +19 %, 48 KiB +2 %, 32 KiB
  // +12 %).  An earlier rule aimed every level at 0.8 rounds (parts of 104 KiB for the 14 ring steps):
  // 227 us against 198-201 us with 64 KiB parts.
  {
    std::vector<long long> level_bytes(n_ops + 1, 0);
    for (int i = 0; i < n_ops; ++i) level_bytes[level[i]] += op_bytes[i];
    parts_by_level.assign(n_ops, 1);
    const long long most_bytes = *std::max_element(level_bytes.begin(), level_bytes.end());
    for (int i = 0; i < n_ops; ++i) {
      if (!G->fixed_parts.empty()) {
        parts[i] = G->fixed_parts[i];
        tiles += parts[i];
        continue;
      }
      long part_bytes = tile_bytes, even_bytes = tile_bytes;
      if (G->want_wide && !G->wide_tile_of.empty()) part_bytes = even_bytes = G->wide_tile_of[i];  // (see wide_cut_of)
      if (default_tile) {
        auto rule = [&](long long bytes) {
          const double want = 16384.0 * std::pow((double)bytes / (double)(8 << 20), 2.0 / 3.0) * (768.0 / (double)cap);
          return (long)std::min<long long>(std::max<long long>(((long long)want + 4095) / 4096 * 4096, 8 << 10), 128 << 10);
        };
        part_bytes = rule(level_bytes[level[i]]);
        even_bytes = rule(most_bytes);
      }
      auto cut = [&](long bytes) {
        long p = (op_bytes[i] + bytes - 1) / bytes;
        if (default_tile) p = std::min<long>(p, (long)cap);
        return (int)std::max<long>(1, std::min<long>(p, kMaxParts));
      };
      parts_by_level[i] = cut(part_bytes);
      parts[i] = cut(even_bytes);  // one size for every level until the chains are known (below): ops of equal length cut alike
      // an op that carries signals of a word per part is cut into as many parts as the signal has words
      if (G->signal_cut[i]) parts_by_level[i] = parts[i] = G->signal_cut[i];
      tiles += parts[i];
    }
    if (tiles > (1ll << 30)) return fail(PCCL_ERR_GRAPH, "graph needs %lld queue entries", tiles);
  }

  // global order of the entries: by level; inside a level the ops by where their predecessors
  // stand in the order (the op whose last predecessor comes first comes first), then op id; the
  // ops of a level take turns with blocks of order_block() consecutive parts.  Workgroups draw tickets in this order and finish their parts at about
  // the pace at which they drew them, so the entry a workgroup draws next should depend on
  // entries that were drawn early.  With op id alone a ring step of rank 0 (which waits for
  // rank 7's previous step, the LAST op of the level before) stood first in its level: ring
  // all-reduce of 8 x 32 MiB 199 -> 195 us, 8 x 8 MiB 88 -> 85 us.  (A list schedule of the graph under a cost model,
  // which lets short chains run ahead of long ones, was measured on the 4096-op schedule and
  // was no faster: workgroups wait longer for dependencies there.)
  std::vector<int> by_level(n_ops);
  for (int i = 0; i < n_ops; ++i) by_level[i] = i;
  std::stable_sort(by_level.begin(), by_level.end(), [&](int a, int b) { return level[a] < level[b]; });
  {
    std::vector<int> last_pred_at(n_ops, -1);  // position of the op's last predecessor in the order
    for (int lo = 0; lo < n_ops;) {
      int hi = lo;
      while (hi < n_ops && level[by_level[hi]] == level[by_level[lo]]) ++hi;
      std::stable_sort(by_level.begin() + lo, by_level.begin() + hi,
                       [&](int a, int b) { return last_pred_at[a] < last_pred_at[b]; });
      for (int at = lo; at < hi; ++at) {
        const int u = by_level[at];
        for (int e = succ_start[u]; e < succ_start[u + 1]; ++e)
          if (succ[e] >= 0) last_pred_at[succ[e]] = std::max(last_pred_at[succ[e]], at);
        for (int v : order_succ[u]) last_pred_at[v] = std::max(last_pred_at[v], at);
      }
      lo = hi;
    }
  }

  // first entry of each op in that order
  std::vector<int> first_entry(n_ops, 0);
  {
    long long t = 0;
    for (int idx = 0; idx < n_ops; ++idx) {
      first_entry[by_level[idx]] = (int)t;
      t += parts[by_level[idx]];
    }
  }

  // ---- dependencies met part by part ---------------------------------------
  // Successor lists again, this time with the successors that are released part by part
  // first, and beside each of those the entry index of its part 0.
  // Each entry then needs a word of its own, 64 bytes from the next (see the arena layout);
  // graphs of more than 4 Mi entries (a 256 MiB array) keep every dependency whole-op.
  G->parts = parts;
  G->part_eligible.assign(n_ops, tiles <= kMaxPartWordEntries);
  G->part_edge = classify_dependencies(G->eff, parts, G->topo, &G->part_eligible);
  // ---- chains (plan_chains) ------------------------------------------------------
  G->n_succ = n_succ;
  G->order_touch.assign(n_ops, 0);
  // (an op that carries a signal op polls or stores a word around its parts: not inside a chain)
  for (int i = 0; i < n_ops; ++i)
    G->order_touch[i] = order_pred[i] != 0 || !order_succ[i].empty() || G->fused_into[i] >= 0 || G->wait_of[i] >= 0 || G->notify_of[i] >= 0;
  G->chain_words = plan_chains_of(G, G->eff, parts, G->part_edge, forward_elem_bytes);
  std::vector<int> chain_prev(n_ops, -1), chain_tail(n_ops, 0);
  auto link_chains = [&] {
    std::fill(chain_prev.begin(), chain_prev.end(), -1);
    for (int i = 0; i < n_ops; ++i) {
      const int nx = G->chain_words[(size_t)kChainWords * i + kChainNext];
      if (nx >= 0) chain_prev[nx] = i;
    }
    for (int i = 0; i < n_ops; ++i) {
      int t = i;
      while (G->chain_words[(size_t)kChainWords * t + kChainNext] >= 0) t = G->chain_words[(size_t)kChainWords * t + kChainNext];
      chain_tail[i] = t;  // (only read for ops that have entries)
    }
  };
  link_chains();
  // A part of a chain costs its workgroup some 20 us whatever its size (every op of the chain waits
  // for the loads and stores of the one before), and the chain's ops queue no entries of their own
  // that could fill the gaps when the resident workgroups finish a round unevenly.  So the built-in
  // choice cuts a level whose entries start chains differently: the smallest part (4 KiB steps from
  // 8 KiB) with which the level's entries fit the resident workgroups once - twice and so on from
  // 96 KiB a part.  Measured on ring all-reduces over 8 virtual ranks, each a chain of 14 ops per
  // rank: 64 MiB 315 us with the 64 KiB parts of the rule above (1.33 rounds), 252 us with 96 KiB
  // (0.9), 264 us with 128 KiB (0.67); 16 MiB 86 -> 79.5 us; 4096-op schedule (288 chains, 64 single ops) 150 -> 133 us.
  if (default_tile && G->fixed_parts.empty()) {
    bool recut = false;
    std::vector<char> settled(n_ops, 0);
    std::vector<std::vector<int>> at_level(n_ops + 1);
    for (int i = 0; i < n_ops; ++i)
      if (chain_prev[i] < 0) at_level[level[i]].push_back(i);
    for (const std::vector<int> &members : at_level) {
      bool heads = false;
      long long bytes = 0;
      for (int i : members) {
        heads = heads || G->chain_words[(size_t)kChainWords * i + kChainNext] >= 0;
        bytes += op_bytes[i];
      }
      if (!heads) continue;
      const long long rounds = std::max<long long>(1, (bytes + (long long)cap * (96 << 10) - 1) / ((long long)cap * (96 << 10)));
      long part_bytes = 8 << 10;
      for (;; part_bytes += 4 << 10) {
        long long entries = 0;
        for (int i : members) entries += std::max<long long>(1, (op_bytes[i] + part_bytes - 1) / part_bytes);
        if (entries <= rounds * (long long)cap || part_bytes >= (1 << 20)) break;
      }
      // Uneven entries (ops of many sizes, most of them too short to cut) leave the round's last
      // workgroups streaming alone: parts of 16 KiB, drawn by ticket in two or three rounds, even that
      // out (4096-op schedule, ops of 8-224 KiB: 98 -> 89 us; uniform ring chunks lose with them).
      if (part_bytes > (16 << 10)) {
        long long entries = 0, longest = 0;
        for (int i : members) {
          const long long n = std::max<long long>(1, (op_bytes[i] + part_bytes - 1) / part_bytes);
          entries += n;
          longest = std::max(longest, (op_bytes[i] + n - 1) / n);
        }
        bool balance = true;
        if (const char *env = getenv("PCCL_HIP_CHAIN_BALANCE")) balance = env[0] != '0';
        if (balance && entries > 0 && longest * entries * 5 > bytes * 6) part_bytes = 16 << 10;  // longest > 1.2 x mean
      }
      for (int i : members) {
        const int p = (int)std::max<long long>(1, std::min<long long>((op_bytes[i] + part_bytes - 1) / part_bytes, cap));
        for (int u = i; u >= 0; u = G->chain_words[(size_t)kChainWords * u + kChainNext]) {
          recut = recut || parts[u] != p;
          parts[u] = p;
          settled[u] = 1;
        }
      }
    }
    for (int i = 0; i < n_ops; ++i)
      if (!settled[i]) {
        recut = recut || parts[i] != parts_by_level[i];
        parts[i] = parts_by_level[i];
      }
    if (recut) {
      tiles = 0;
      for (int i = 0; i < n_ops; ++i) tiles += parts[i];
      long long t = 0;
      for (int idx = 0; idx < n_ops; ++idx) {
        first_entry[by_level[idx]] = (int)t;
        t += parts[by_level[idx]];
      }
      G->parts = parts;
      G->part_eligible.assign(n_ops, tiles <= kMaxPartWordEntries);
      G->part_edge = classify_dependencies(G->eff, parts, G->topo, &G->part_eligible);
      G->chain_words = plan_chains_of(G, G->eff, parts, G->part_edge, forward_elem_bytes);
      link_chains();
    }
  }
  auto queued = [&](int i) { return chain_prev[i] < 0 && G->fused_into[i] < 0; };  // has entries of its own
  long long live_tiles = 0;
  for (int i = 0; i < n_ops; ++i)
    if (queued(i)) live_tiles += parts[i];
  // The wide launch (wide_body) is open to a graph none of whose entries waits for another entry (as
  // for entries without tickets, below) or has to do with a signal word (its workgroups poll nothing
  // and tell nobody), with no more entries than kMaxWideEntries (40 bytes of arena each).
  {
    bool waits = carries;
    for (int i = 0; i < n_ops && !waits; ++i)
      waits = queued(i) && (n_pred[i] > 0 || order_pred[i] > 0 || ops[i].primitive == PCCL_NOTIFY || ops[i].primitive == PCCL_GET_NOTIFIED);
    G->wide_ok = !waits && live_tiles > 0 && live_tiles <= kMaxWideEntries;
    // (what the entries that do not run a chain in one pass move, chains through memory included: see wide_launch_pays)
    G->wide_plain_bytes = 0;
    G->wide_plain_streams = 0;
    G->wide_chain_bytes = 0;
    G->wide_slow = false;
    for (int i = 0; i < n_ops; ++i) {
      if (!queued(i)) continue;
      const int *w = &G->chain_words[(size_t)kChainWords * i];
      if (w[kChainNext] >= 0 && w[kChainForward] == 1) {
        for (int u = i, k = 0; u >= 0 && k < w[kChainLength]; u = G->chain_words[(size_t)kChainWords * u + kChainNext], ++k)
          G->wide_chain_bytes += (long long)(ops[u].n_in + ops[u].n_out) * op_bytes[u];
        continue;
      }
      int steps = 0;  // ops of the chain that run (a copy that its producer stores does not)
      for (int u = i; u >= 0; u = G->chain_words[(size_t)kChainWords * u + kChainNext]) {
        G->wide_plain_bytes += (long long)(ops[u].n_in + ops[u].n_out) * op_bytes[u];
        const int after = G->chain_words[(size_t)kChainWords * u + kChainNext];
        const bool stores_next = after >= 0 && G->chain_words[(size_t)kChainWords * after + kChainForward] == kChainFolded;
        G->wide_plain_streams = std::max(G->wide_plain_streams, ops[u].n_in + ops[u].n_out + (stores_next ? ops[after].n_out : 0));
        if (G->chain_words[(size_t)kChainWords * u + kChainForward] != kChainFolded || u == i) ++steps;
      }
      // A long chain through memory is a row of dependent round trips per workgroup (stores acknowledged,
      // barrier, next op's loads), which the drain's longer parts carry better than short-lived workgroups:
      // one rank's 14 ring steps as one such chain 209 us through the drain, 247 us wide.
      if (steps > 2) G->wide_slow = true;
    }
    if (G->want_wide && (!G->wide_ok || (G->fixed_n_wg > 0 && live_tiles > G->fixed_n_wg)))
      return fail(PCCL_ERR_UNSUPPORTED, "with these operands the graph does not run as a wide launch (an entry waits for another, "
                                        "or there are more entries than the launch was made for)");
  }
  // A wide launch of at most kMaxLaunchChains entries that are each one fold runs in the shape of the
  // direct kernels instead (graph_chains_device.h), with the direct launch's rules for one launch of all
  // this traffic (reduce_copy.hip): streaming treatment and chunk rotation from 48 MiB in all, an
  // occupancy cap beyond the Infinity Cache.
  std::vector<LaunchChain> launch_rows;
  int launch_shape = 0;
  G->chains_launch = false;
  if (G->want_wide && !mixed && (G->fixed_chains ? G->fixed_chains->chains_launch : chain_launch_mode() != 0) &&
      launch_chains_of(G->eff, G->chain_words, g_dtype, g_compute, &launch_rows, &launch_shape)) {
    ChainsLaunch &a = G->chains_args;
    memset(&a, 0, sizeof(a));
    long long blocks = 0, total_bytes = 0;
    int streams = 1;
    bool folds = false;
    a.n_chains = (int)launch_rows.size();
    a.group = (a.n_chains + kLaunchChainGroups - 1) / kLaunchChainGroups;
    for (int k = 0; k < kLaunchChainGroups; ++k) a.first_wg[k] = 0xffffffffu;
    for (size_t k = 0; k < launch_rows.size(); ++k) {
      LaunchChain &c = launch_rows[k];
      c.first_wg = (unsigned int)blocks;
      if (k % (size_t)a.group == 0) a.first_wg[k / (size_t)a.group] = c.first_wg;
      blocks += c.n_wg;
      total_bytes += (long long)(c.n_in + c.n_out) * c.count * elem_bytes(g_dtype);
      streams = std::max(streams, c.n_in + c.n_out);
      folds = folds || c.n_in > 1;
    }
    const bool pays = (launch_shape & kChainsFold) || ((launch_shape & kChainsFanOut) && total_bytes >= (48ll << 20));
    if (blocks < (1ll << 31) && (pays || G->fixed_chains || chain_launch_mode() == 2)) {
      G->chains_launch = true;
      G->chains_grid = (unsigned)blocks;
      G->chains_mem = total_bytes >= (48ll << 20) ? (int)kLaunchMemStreamWriteThrough : (int)kLaunchMemCached;
      if (G->chains_mem && (launch_shape & kChainsFanOut)) G->chains_mem = kLaunchMemStream;  // (as a direct launch treats a copy to three or more outputs)
      a.rotate = G->chains_mem != 0;
      G->chains_lds = 0;
      if (total_bytes > (192ll << 20)) {
        int wgs = std::max(2, std::min(8, (20 + streams / 2) / streams));
        if (elem_bytes(g_dtype) == 1 && folds) wgs = std::max(wgs, 4);
        if (wgs < 8) G->chains_lds = std::min(65536u, (unsigned)(160 * 1024 / wgs) - 256u);
      }
      G->chains_dtype = g_dtype;
      G->chains_compute = g_compute;
      G->chains_kernel = chains_kernel_for(g_dtype, g_compute, G->chains_mem);
    }
  }
  if (const Graph *F = G->fixed_chains) {
    // (launches that a stream capture has recorded carry the kernel, the grid and the arguments)
    const bool same = F->chains_launch == G->chains_launch &&
                      (!F->chains_launch || (F->chains_grid == G->chains_grid && F->chains_lds == G->chains_lds && F->chains_kernel == G->chains_kernel &&
                                             F->chains_args.rotate == G->chains_args.rotate && F->chains_args.group == G->chains_args.group &&
                                             F->chains_args.n_chains == G->chains_args.n_chains &&
                                             !memcmp(F->chains_args.first_wg, G->chains_args.first_wg, sizeof(F->chains_args.first_wg))));
    if (!same)
      return fail(PCCL_ERR_UNSUPPORTED, "with these operands the graph does not run as the launch it was made for (its chains come out differently)");
  }

  std::vector<int> succ_part_base(n_edges ? n_edges : 1, -1), n_part_next(n_ops, 0), n_part_pred(n_ops, 0);
  {
    size_t at = 0;
    for (int i = 0; i < n_ops; ++i)
      for (int d = 0; d < ops[i].n_deps; ++d, ++at)
        if (G->part_edge[at]) {
          ++n_part_next[ops[i].deps[d]];
          ++n_part_pred[i];
        }
    std::vector<int> fill_part(n_ops, 0), fill_whole(n_ops, 0);
    at = 0;
    for (int i = 0; i < n_ops; ++i)
      for (int d = 0; d < ops[i].n_deps; ++d, ++at) {
        const int u = ops[i].deps[d];
        const int pos = succ_start[u] + (G->part_edge[at] ? fill_part[u]++ : n_part_next[u] + fill_whole[u]++);
        succ[pos] = i;
        succ_part_base[pos] = G->part_edge[at] ? first_entry[i] : -1;
      }
  }

  // ---- arena layout ----------------------------------------------------------
  size_t off = align_up(sizeof(GraphControl), 256);
  const size_t off_opptr = off;   off = align_up(off + sizeof(void *) * (size_t)std::max(n_ops, 1), 256);
  const size_t off_hdr = off;     off = align_up(off + sizeof(pccl_operation_layout_header) * (size_t)std::max(n_ops, 1), 256);
  const size_t off_payload = off; off = align_up(off + kPayloadStride * (size_t)std::max(n_ops, 1), 256);
  // (the chain table follows the payloads directly: graph_rebind uploads the two as one block)
  const size_t off_chain_table = off; off = off + sizeof(ForwardStep) * (size_t)std::max(n_ops, 1);
  // (... and the table of carried signals directly behind that one, for the same reason)
  const size_t off_fuse = off;        off = align_up(off + sizeof(SignalFuse) * (size_t)std::max(n_ops, 1), 256);
  const size_t off_succ = off;    off = align_up(off + sizeof(int) * std::max<size_t>(n_edges, 1), 256);
  const size_t off_succ_part = off; off = align_up(off + sizeof(int) * std::max<size_t>(n_edges, 1), 256);
  const size_t off_hot = off;     off = align_up(off + sizeof(HotWord) * kHotWords, 256);
  int n_grouped = 0;  // ops that count their parts in groups
  for (int i = 0; i < n_ops; ++i) n_grouped += parts[i] > kGroupThreshold;
  const size_t off_ready = off;   off = align_up(off + sizeof(HotWord) * (size_t)std::max(n_ops, 1), 256);
  const size_t off_gbase = off;   off = align_up(off + sizeof(int) * (size_t)std::max(n_ops, 1), 256);
  const size_t off_ebase = off;   off = align_up(off + sizeof(int) * (size_t)std::max(n_ops, 1), 256);
  const size_t off_groups = off;  off = align_up(off + sizeof(HotWord) * (size_t)kPartGroups * (size_t)std::max(n_grouped, 1), 256);
  const size_t off_chain = off;   off = align_up(off + kChainWords * sizeof(int) * (size_t)std::max(n_ops, 1), 256);
  // One word per entry, 64 bytes apart: a word is polled by the workgroup that holds its entry
  // and bumped by others.  Packed 32 to a 128-byte line they cost more than the part-by-part
  // hand-over saves (ring all-reduce of 8 x 1 MiB: 82 us against 76 us with whole-op waits;
  // 64 bytes apart: 66 us; 8 x 8 MiB: 114 -> 94 us against 123; the 4096-op schedule 181 -> 171 us).
  // The words are there whether or not a dependency uses them now: graph_rebind can change
  // that, and must not change the arena's layout.
  const size_t off_part_arrivals = off;
  const int part_shift = 4;
  const bool part_words = tiles <= kMaxPartWordEntries;
  if (part_words) off = align_up(off + (sizeof(unsigned int) << part_shift) * (size_t)(tiles + kQueues), 256);
  const size_t off_ring = off;    off = align_up(off + 256 * (size_t)kQueues, 256);  // one RingBuffer per 256-byte line
  const size_t off_qptr = off;    off = align_up(off + sizeof(void *) * kQueues, 256);
  const size_t off_qcount = off;  off = align_up(off + sizeof(int) * (kQueues + 1), 256);  // queue lengths, mode word
  // room for an entry per part of every op, an equal share per queue: where the queues start must not
  // depend on how many entries the chains leave to be queued (graph_rebind can change that)
  const size_t queue_room = (size_t)((std::max<long long>(tiles, 1) + kQueues - 1) / kQueues);
  const size_t off_entries = off; off = align_up(off + 8 * queue_room * kQueues, 256);
  // (a wide launch: a record per workgroup; room for one per part of every op, so that the layout does not move with the chain plan)
  const size_t off_wide = off;    if (G->want_wide) off = align_up(off + sizeof(WideEntry) * (size_t)std::max<long long>(tiles, 1), 256);
  const size_t off_lchains = off; if (G->want_wide) off = align_up(off + sizeof(LaunchChain) * (size_t)kMaxLaunchChains, 256);
  const size_t arena_bytes = off;

  G->n_ops = n_ops;
  // entries that are queued (the arena has room for an entry per part of every op); a launch of chains: its workgroups, which is what a trace records
  G->total_tiles = (int)(G->chains_launch ? (long long)G->chains_grid : live_tiles);
  G->all_tiles = (int)std::max<long long>(tiles, G->total_tiles);
  G->payload_off = off_payload;
  G->kernel_elem_bytes = elem_bytes(g_dtype);
  if (G->fixed_kernel) {
    G->kernel = G->fixed_kernel;
  } else {
    G->forward_capable = false;
    for (int i = 0; i < n_ops && forward_kernel; ++i)
      if (chain_prev[i] < 0 && G->chain_words[(size_t)kChainWords * i + kChainNext] >= 0 && G->chain_words[(size_t)kChainWords * i + kChainForward])
        G->forward_capable = true;
    G->kernel = G->forward_capable ? forward_kernel : plain_kernel;
  }
  if (hipGetDevice(&G->device) != hipSuccess) return fail(PCCL_ERR_NO_DEVICE, "no current device");
  G->dev = nullptr;
  G->arena_bytes = arena_bytes;
  hipError_t e = hipSuccess;
  if (fixed) {
    if (arena_bytes > fixed->capacity)
      return fail(PCCL_ERR_NOMEM, "the op graph needs %zu bytes of device state; the static arena holds %zu "
                                  "(%d ops, %lld queue entries)", arena_bytes, fixed->capacity, n_ops, tiles);
    G->dev = fixed->ptr;
  } else if (reuse && reuse_bytes == arena_bytes) G->dev = reuse;
  else e = hipMalloc((void **)&G->dev, arena_bytes);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    G->dev = nullptr;
    return fail(PCCL_ERR_NOMEM, "hipMalloc(%zu) for the op graph: %s", arena_bytes, hipGetErrorString(e));
  }
  G->image.assign(arena_bytes, 0);
  char *img = G->image.data();
  char *dev = G->dev;

  GraphControl *C = (GraphControl *)img;
  HotWord *hot = (HotWord *)(img + off_hot);
  C->hot = (HotWord *)(dev + off_hot);
  C->layout.completed_operator = &((HotWord *)(dev + off_hot))[kHotCompleted].value;
  C->layout.total_operator = &((HotWord *)(dev + off_hot))[kHotTotal].value;
  C->layout.operators = (pccl_operation_layout_header **)(dev + off_opptr);
  C->layout.num_operators = (unsigned int)n_ops;
  C->layout.ready_queues = (pccl_ring_buffer **)(dev + off_qptr);
  C->layout.num_queues = kQueues;
  C->headers = (pccl_operation_layout_header *)(dev + off_hdr);
  C->slots = dev + off_payload;
  C->succ = (const int *)(dev + off_succ);
  C->succ_part_base = (const int *)(dev + off_succ_part);
  C->part_arrivals = part_words ? (unsigned int *)(dev + off_part_arrivals) : nullptr;
  C->part_shift = part_shift;
  C->trace = G->trace_on ? G->trace : nullptr;
  C->group_base = (const int *)(dev + off_gbase);
  C->entry_base = (const int *)(dev + off_ebase);
  for (int i = 0; i < n_ops; ++i) ((int *)(img + off_ebase))[i] = first_entry[i];
  C->groups = (HotWord *)(dev + off_groups);
  C->ready = (HotWord *)(dev + off_ready);
  {
    int *gbase = (int *)(img + off_gbase);
    HotWord *groups = (HotWord *)(img + off_groups);
    int next = 0;
    for (int i = 0; i < n_ops; ++i) {
      gbase[i] = -1;
      if (parts[i] <= kGroupThreshold) continue;
      gbase[i] = next;
      for (int k = 0; k < kPartGroups; ++k) groups[next + k].value = (unsigned int)((parts[i] - k + kPartGroups - 1) / kPartGroups);
      next += kPartGroups;
    }
  }
  C->spin_limit = G->spin_limit;
  C->n_ops = (unsigned int)n_ops;
  C->wide_entries = G->want_wide ? (const WideEntry *)(dev + off_wide) : nullptr;
  G->chains_off = off_lchains;
  if (G->chains_launch) {
    memcpy(img + off_lchains, launch_rows.data(), sizeof(LaunchChain) * launch_rows.size());
    G->chains_args.chains = (const LaunchChain *)(dev + off_lchains);
  }
  C->queue_count = (const int *)(dev + off_qcount);
  C->chain = (const int *)(dev + off_chain);
  C->chain_table = (const ForwardStep *)(dev + off_chain_table);
  G->chain_table_off = off_chain_table;
  G->fuse_table_off = off_fuse;
  C->fuse = (const SignalFuse *)(dev + off_fuse);
  memcpy(img + off_chain, G->chain_words.data(), sizeof(int) * G->chain_words.size());
  hot[kHotCompleted].value = 0;
  hot[kHotTotal].value = (unsigned int)n_ops;
  hot[kHotRun].value = run_number;

  // deal the entries round-robin onto the queues, in global order
  std::vector<std::vector<unsigned long long>> qe(kQueues);
  {
    long long t = 0;
    // (a wide launch: op after op, so that the workgroups in flight cover few ops at a time, each through
    // a narrow window like a direct launch: ring all-reduce 8 x 64 MiB 212 -> 196 us, 8 x 32 MiB 90.6 -> 88.8)
    const int block = G->want_wide ? 1 << 30 : order_block();
    WideEntry *wide_entries = G->want_wide ? (WideEntry *)(img + off_wide) : nullptr;
    // (PCCL_HIP_COUNT_ALL=1: also the parts of ops that nobody waits for are counted, see kEntryUncounted)
    const char *count_env = getenv("PCCL_HIP_COUNT_ALL");
    const int count_all_parts = count_env && count_env[0] == '1';
    for (int lo = 0; lo < n_ops;) {
      int hi = lo, most = 0;
      while (hi < n_ops && level[by_level[hi]] == level[by_level[lo]]) most = std::max(most, parts[by_level[hi++]]);
      std::vector<int> turn(by_level.begin() + lo, by_level.begin() + hi);
      int step = block;
      if (hi == n_ops && lo > 0 && last_level_longest_first()) {
        // The last level of several: its entries are the last ones drawn, and the run ends when the last
        // of them does.  Op after op, the ops whose parts move most bytes first, so that the entries the
        // run ends with are the short ones.
        // (in half octaves of streams x bytes per part: ops cut to about the same part keep their order)
        auto cost = [&](int i) {
          const double bytes = (double)(ops[i].n_in + ops[i].n_out) * (double)part_elems(ops[i].count, std::max(1, parts[i])) * elem_bytes(ops[i].dtype);
          return (int)std::lround(2.0 * std::log2(std::max(1.0, bytes)));
        };
        std::stable_sort(turn.begin(), turn.end(), [&](int a, int b) { return cost(a) > cost(b); });
        step = 1 << 30;
      }
      for (int first = 0; first < most; first += step)
        for (int i : turn) {
          if (!queued(i)) continue;  // runs behind its chain's head
          for (int p = first; p < (int)std::min<long long>((long long)first + step, parts[i]); ++p, ++t) {
            if (wide_entries) {
              const long per = part_elems(ops[i].count, parts[i]), lo = (long)p * per;
              WideEntry &w = wide_entries[t];
              w.uid = i;
              w.n = (int)std::max<long>(0, std::min<long>(per, ops[i].count - lo));
              w.lo = lo;
              for (int k = 0; k < kChainWords; ++k) w.chain[k] = G->chain_words[(size_t)kChainWords * i + k];
            }
            qe[t % kQueues].push_back((unsigned long long)(unsigned int)i | ((unsigned long long)p << 32) |
                                      ((G->chain_words[(size_t)kChainWords * i + kChainNext] >= 0 || G->wait_of[i] >= 0 || G->notify_of[i] >= 0) ? kEntryChainHead : 0ull) |
                                      (G->wait_of[i] >= 0 ? kEntryWaitsSignal : 0ull) | (notifies_by_part(i) ? kEntryNotifiesPart : 0ull) |
                                      ((count_all_parts == 0 && n_succ[chain_tail[i]] == 0 && n_pred[i] == n_part_pred[i]) ? kEntryUncounted : 0ull));
          }
        }
      lo = hi;
    }
  }
  {
    for (int q = 0; q < kQueues; ++q) {
      const size_t pos = off_entries + 8 * queue_room * (size_t)q;
      ((pccl_ring_buffer **)(img + off_qptr))[q] = (pccl_ring_buffer *)(dev + off_ring + 256 * (size_t)q);
      pccl_ring_buffer *R = (pccl_ring_buffer *)(img + off_ring + 256 * (size_t)q);
      C->queue_head[q] = &((pccl_ring_buffer *)(dev + off_ring + 256 * (size_t)q))->head_;
      C->queue_entries[q] = (const unsigned long long *)(dev + pos);
      ((int *)(img + off_qcount))[q] = (int)qe[q].size();
      R->producer_ = (pccl_general_type)pccl_host::executor_id();  // one executor fills and drains
      R->consumer_ = (pccl_general_type)pccl_host::executor_id();
      R->elem_size_ = (int)sizeof(pccl_queue_entry);
      R->max_num_elems_ = (int)qe[q].size();
      R->max_flush_time_ = 0;  // producer and consumer share one address space: nothing to flush
      R->tail_ = (int)qe[q].size();
      R->head_ = 0;
      R->producer_buffer_ = dev + pos;
      R->consumer_buffer_ = dev + pos;
      if (!qe[q].empty()) memcpy(img + pos, qe[q].data(), 8 * qe[q].size());
    }
  }

  for (int i = 0; i < n_ops; ++i) {
    const pccl_op_desc &o = ops[i];
    ((pccl_operation_layout_header **)(img + off_opptr))[i] =
        (pccl_operation_layout_header *)(dev + off_hdr) + i;
    pccl_operation_layout_header *h = (pccl_operation_layout_header *)(img + off_hdr) + i;
    h->op_uid_ = i;
    h->required_executors_ = parts[i];
    h->remaining_executors_ = parts[i] > kGroupThreshold ? kPartGroups : parts[i];
    h->pre_dependencies_ = (unsigned char)n_pred[i];
    h->executor_type_ = (pccl_general_type)pccl_host::executor_id();
    h->op_size_ = (unsigned char)(8 + sizeof(pccl_chunk_meta) * (size_t)(o.n_in + o.n_out));
    h->num_next_ops_ = (unsigned char)n_succ[i];
    h->op_buffer_ = dev + off_payload + kPayloadStride * (size_t)i;
    h->next_op_uids_head_ = (int *)(dev + off_succ) + succ_start[i];
    PayloadSlot *slot = (PayloadSlot *)(img + off_payload + kPayloadStride * (size_t)i);
    const int tail = chain_tail[i];  // (the op itself unless it heads a chain)
    slot->parts = parts[i];
    slot->succ_start = succ_start[tail];
    pccl_op_payload *pl = &slot->payload;
    pl->primitive_ = o.primitive;
    pl->compute_ = o.compute;
    pl->n_in_ = o.n_in;
    pl->n_out_ = o.n_out;
    pl->pre_dependencies_ = h->pre_dependencies_;
    pl->part_preds_ = (unsigned char)n_part_pred[i];
    pl->part_nexts_ = (unsigned char)n_part_next[tail];
    pl->num_next_ops_ = (unsigned char)n_succ[tail];
    // signal ops: the only operand is the signal word, num_elems_ carries the value
    for (int k = 0; k < o.n_in; ++k) pl->chunks_[k] = pccl_chunk_meta{o.dtype, (void *)o.ins[k], o.count};
    for (int k = 0; k < o.n_out; ++k) pl->chunks_[o.n_in + k] = pccl_chunk_meta{o.dtype, o.outs[k], o.count};
    if (o.primitive == PCCL_NOTIFY || o.primitive == PCCL_GET_NOTIFIED) {
      // ... and behind it the number of words the signal has (one, or one per part)
      pl->chunks_[1] = pccl_chunk_meta{o.dtype, nullptr, o.signal_parts >= 2 ? (long)o.signal_parts : 1l};
      h->op_size_ = (unsigned char)(8 + sizeof(pccl_chunk_meta) * 2);
    }
  }
  fill_chain_table(G->chain_words, n_ops, img + off_payload, (ForwardStep *)(img + off_chain_table));
  fill_fuse_table(G, G->eff, (SignalFuse *)(img + off_fuse));
  if (n_edges) memcpy(img + off_succ, succ.data(), sizeof(int) * n_edges);
  if (n_edges) memcpy(img + off_succ_part, succ_part_base.data(), sizeof(int) * n_edges);
  // never more workgroups than entries
  // (a rebuild in place keeps the count: launches that a stream capture has recorded carry it)
  G->n_wg = G->fixed_n_wg > 0 ? G->fixed_n_wg : (int)std::max<long long>(1, std::min<long long>(live_tiles, G->want_wide ? kMaxWideEntries : cap));
  if (G->chains_launch) G->n_wg = (int)G->chains_grid;
  G->wide = G->want_wide;
  {
    // Entries without tickets (graph_queue_device.h): when there is at most one per workgroup
    // (PCCL_HIP_OWN_ENTRIES=k: up to k; the mapping of entries to workgroups then needs every queue to
    // have the same number of workgroups) AND no queued entry waits for another entry of this graph.
    // An entry that belongs to a workgroup by number can belong to one that has no compute unit yet;
    // whoever waits for it then waits for the dispatcher, which hands out a launch's workgroups in
    // order per XCD but shares the compute units with whatever else runs: beside a second graph of
    // this kind (or any kernel that does not end by itself) the two can hold each other's compute
    // units while the entries they wait for sit with workgroups that cannot start.  Tickets have no
    // such case (only a running workgroup ever holds an entry), so graphs whose entries depend on
    // each other draw tickets; chains' heads, independent ops and waits for signals from outside the
    // graph depend on no other entry.
    long long rounds = 1;
    if (const char *env = getenv("PCCL_HIP_OWN_ENTRIES")) rounds = atoll(env);
    bool entries_wait = false;
    for (int i = 0; i < n_ops && !entries_wait; ++i)
      entries_wait = queued(i) && (n_pred[i] > 0 || order_pred[i] > 0);
    const bool own = rounds > 0 && !entries_wait &&
                     (live_tiles <= (long long)G->n_wg ||
                      (G->n_wg % kQueues == 0 && live_tiles <= rounds * (long long)G->n_wg));
    ((int *)(img + off_qcount))[kQueues] = own ? 1 : 0;
  }

  e = fixed ? hipMemcpyAsync(dev, img, arena_bytes, hipMemcpyHostToDevice, fixed->stream)
            : hipMemcpy(dev, img, arena_bytes, hipMemcpyHostToDevice);
  if (e != hipSuccess) {
    if (dev != reuse && !fixed) (void)hipFree(dev);
    G->dev = nullptr;
    return fail(PCCL_ERR_HIP, "uploading the op graph: %s", hipGetErrorString(e));
  }
  return PCCL_OK;
}

// ---- the arena of pccl_hip_graph_run_static ---------------------------------------
// Device state of ONE op graph per GPU in a file-scope device array, for callers that cannot
// allocate device memory.  On the host the array's name is only a handle: its address on a
// device comes from hipGetSymbolAddress (once per device, that device current) and only that
// address is ever handed to a kernel or a copy.
constexpr size_t kStaticArenaBytes = PCCL_HIP_STATIC_ARENA_BYTES;
constexpr int kMaxStaticDevices = 64;
struct StaticArena {
  char *ptr = nullptr;          // this device's copy of g_static_arena
  Graph *graph = nullptr;       // host side of what the array holds now
  bool valid = false;           // ... and it is complete and was not left behind by an aborted run
  bool used = false;
  bool launched = false;        // a drain kernel has run on the state the array holds now
  hipStream_t last_stream = nullptr;
  unsigned int runs = 0;        // launches on this array so far (signal values go on from here)
  std::vector<int> deps;        // the call's dependency lists, back to back (kept between calls: no host allocation once it has grown)
};
std::mutex g_static_mutex;
StaticArena g_static[kMaxStaticDevices];

}  // namespace

static __device__ __align__(256) unsigned char g_static_arena[PCCL_HIP_STATIC_ARENA_BYTES];

extern "C" {

int pccl_hip_graph_create(const pccl_op_desc *ops, int n_ops, long tile_bytes, void **graph) {
  pccl_host::clear_error();
  if (!graph) return fail(PCCL_ERR_INVALID_ARG, "graph_create: graph is null");
  *graph = nullptr;
  if (n_ops < 0 || (n_ops > 0 && !ops)) return fail(PCCL_ERR_INVALID_ARG, "graph_create: bad op array");
  if (tile_bytes < 0 && tile_bytes != PCCL_HIP_TILE_AUTO) return fail(PCCL_ERR_INVALID_ARG, "graph_create: tile_bytes %ld < 0", tile_bytes);
  const bool may_plan = tile_bytes == PCCL_HIP_TILE_AUTO;
  if (may_plan) tile_bytes = 0;
  // own copy of the ops and their dependency lists
  Graph *G = new Graph();
  G->tile_bytes = tile_bytes;
  G->spin_limit = default_spin_limit();
  G->descs.assign(ops, ops + n_ops);
  size_t n_deps = 0;
  for (int i = 0; i < n_ops; ++i) {
    if (ops[i].n_deps < 0 || (ops[i].n_deps > 0 && !ops[i].deps)) {
      delete G;
      return fail(PCCL_ERR_GRAPH, "op %d: bad dependency list", i);
    }
    n_deps += (size_t)ops[i].n_deps;
  }
  G->deps_store.reserve(n_deps);
  for (int i = 0; i < n_ops; ++i) G->deps_store.insert(G->deps_store.end(), ops[i].deps, ops[i].deps + ops[i].n_deps);
  for (int i = 0, at = 0; i < n_ops; at += ops[i].n_deps, ++i) G->descs[i].deps = G->deps_store.data() + at;
  if (may_plan && plan_launches(G->descs, &G->launches)) {
    // the launches' operands are checked now, as graph_create checks a queue graph's
    for (const pccl_op_desc &o : G->launches) {
      const int rc = check_launch(o);
      if (rc != PCCL_OK) {
        delete G;
        return rc;
      }
    }
    G->as_launches = true;
    G->n_ops = n_ops;
    if (hipGetDevice(&G->device) != hipSuccess) {
      delete G;
      return fail(PCCL_ERR_NO_DEVICE, "no current device");
    }
    *graph = G;
    return PCCL_OK;
  }
  const int rc = build_graph(G, 1);
  if (rc != PCCL_OK) {
    delete G;
    return rc;
  }
  // The library's own cut (tile_bytes 0): a graph whose entries wait for nothing runs as a wide launch
  // (wide_body), for which it is cut again, every op into parts of one block.  If that cut does not
  // keep the property (or its arena cannot be had), the graph stays as built.
  if (G->tile_bytes == 0 && G->wide_ok && !G->wide_slow && wide_launch_pays()) {
    Graph *W = new Graph();
    W->tile_bytes = 0;
    W->spin_limit = G->spin_limit;
    W->descs = G->descs;
    W->deps_store = G->deps_store;
    for (int i = 0, at = 0; i < n_ops; at += ops[i].n_deps, ++i) W->descs[i].deps = W->deps_store.data() + at;
    W->want_wide = true;
    wide_cut_of(G, W);
    if (build_graph(W, 1) == PCCL_OK) {
      if (G->dev) (void)hipFree(G->dev);
      delete G;
      G = W;
    } else {
      delete W;
      pccl_host::clear_error();
    }
  }
  *graph = G;
  return PCCL_OK;
}

int pccl_hip_graph_run(void *graph, void *stream) {
  pccl_host::clear_error();
  Graph *G = (Graph *)graph;
  if (!G) return fail(PCCL_ERR_INVALID_ARG, "graph_run: graph is null");
  // (a launch goes to the calling thread's current device, the graph's memory lives on the one it was created on)
  int current = -1;
  if (hipGetDevice(&current) != hipSuccess || current != G->device)
    return fail(PCCL_ERR_INVALID_ARG, "graph_run: the graph was created on device %d, the current device is %d", G->device, current);
  if (G->as_launches) {
    std::vector<pccl_op_desc> launches;
    {
      std::lock_guard<std::mutex> lock(G->mu);  // graph_rebind may be moving operands
      launches = G->launches;
    }
    for (const pccl_op_desc &o : launches) {
      const int rc = pccl_hip_reduce_copy(o.dtype, o.compute, o.ins, o.n_in, o.outs, o.n_out, o.count, stream);
      if (rc != PCCL_OK) return rc;
    }
    std::lock_guard<std::mutex> lock(G->mu);
    ++G->runs;
    return PCCL_OK;
  }
  if (G->total_tiles == 0) return PCCL_OK;
  GraphControl control;
  ChainsLaunch args;
  {
    std::lock_guard<std::mutex> lock(G->mu);  // spin_limit may be changed by another thread
    memcpy(&control, G->image.data(), sizeof(control));
    args = G->chains_args;
  }
  if (G->chains_launch) {
    args.trace = control.trace;
    hipLaunchKernelGGL(G->chains_kernel, dim3(G->chains_grid), dim3(kBlock), G->chains_lds, (hipStream_t)stream, args);
  } else {
    hipLaunchKernelGGL(G->kernel, dim3((unsigned)G->n_wg), dim3(kBlock), G->wide ? G->wide_lds : 0u, (hipStream_t)stream, control);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(PCCL_ERR_HIP, "graph_run launch failed: %s", hipGetErrorString(e));
  {
    // counted only once the launch is in: the device's run word moves on per executed launch
    std::lock_guard<std::mutex> lock(G->mu);
    ++G->runs;
  }
  return PCCL_OK;
}

int pccl_hip_graph_trace(void *graph, int enable) {
  pccl_host::clear_error();
  Graph *G = (Graph *)graph;
  if (!G) return fail(PCCL_ERR_INVALID_ARG, "graph_trace: graph is null");
  if (G->as_launches) return fail(PCCL_ERR_UNSUPPORTED, "graph_trace: this graph runs as %zu plain launches, there are no queue entries to time", G->launches.size());
  std::lock_guard<std::mutex> lock(G->mu);
  GraphControl *C = (GraphControl *)G->image.data();
  G->trace_on = enable != 0;
  if (!enable) { C->trace = nullptr; return PCCL_OK; }  // the buffer stays until the graph is destroyed
  // (room for a record per part of every op: a rebind may change how many of them are queued)
  const size_t bytes = sizeof(unsigned long long) * kTraceWords * (size_t)std::max(G->all_tiles, 1);
  if (!G->trace) {
    hipError_t e = hipMalloc((void **)&G->trace, bytes);
    if (e != hipSuccess) {
      (void)hipGetLastError();
      G->trace = nullptr;
      return fail(PCCL_ERR_NOMEM, "hipMalloc(%zu) for the trace records: %s", bytes, hipGetErrorString(e));
    }
  }
  PCCL_HIP_CHECK(hipMemset(G->trace, 0, bytes));
  C->trace = G->trace;
  return PCCL_OK;
}

int pccl_hip_graph_read_trace(void *graph, void *stream, unsigned long long *records, long capacity, long *n_records) {
  pccl_host::clear_error();
  Graph *G = (Graph *)graph;
  if (!G || !n_records) return fail(PCCL_ERR_INVALID_ARG, "graph_read_trace: null argument");
  *n_records = 0;
  if (!G->trace) return fail(PCCL_ERR_INVALID_ARG, "graph_read_trace: tracing was never switched on for this graph");
  if (capacity < 0 || (capacity > 0 && !records)) return fail(PCCL_ERR_INVALID_ARG, "graph_read_trace: bad record buffer");
  PCCL_HIP_CHECK(hipStreamSynchronize((hipStream_t)stream));
  const long n = std::min<long>(capacity, G->total_tiles);
  if (n > 0)
    PCCL_HIP_CHECK(hipMemcpy(records, G->trace, sizeof(unsigned long long) * kTraceWords * (size_t)n, hipMemcpyDeviceToHost));
  *n_records = G->total_tiles;
  return PCCL_OK;
}

int pccl_hip_graph_status(void *graph, void *stream, unsigned int *completed, unsigned int *total) {
  pccl_host::clear_error();
  Graph *G = (Graph *)graph;
  if (!G) return fail(PCCL_ERR_INVALID_ARG, "graph_status: graph is null");
  PCCL_HIP_CHECK(hipStreamSynchronize((hipStream_t)stream));
  if (G->as_launches || G->wide) {  // launches that have ended have completed their ops (nothing in them waits)
    if (completed) *completed = G->runs ? (unsigned int)G->n_ops : 0u;
    if (total) *total = (unsigned int)G->n_ops;
    return PCCL_OK;
  }
  const size_t off_hot = (size_t)((const char *)((const GraphControl *)G->image.data())->hot - G->dev);
  HotWord hot[kHotWords];
  PCCL_HIP_CHECK(hipMemcpy(hot, G->dev + off_hot, sizeof(hot), hipMemcpyDeviceToHost));
  if (completed) *completed = hot[kHotCompleted].value;
  if (total) *total = hot[kHotTotal].value;
  if (hot[kHotAbort].value) {
    // put the pristine state back so that the graph can be used again
    std::lock_guard<std::mutex> lock(G->mu);
    PCCL_HIP_CHECK(hipMemcpy(G->dev, G->image.data(), G->image.size(), hipMemcpyHostToDevice));
    // ... except the run number, which the aborted run has already moved on
    PCCL_HIP_CHECK(hipMemcpy(G->dev + off_hot + sizeof(HotWord) * kHotRun, &hot[kHotRun], sizeof(HotWord),
                             hipMemcpyHostToDevice));
    return fail(PCCL_ERR_GRAPH, "drain gave up: an op's dependencies were not satisfied within the spin limit "
                                "(%u of %u ops had completed); graph state was reset",
                hot[kHotCompleted].value, hot[kHotTotal].value);
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
  auto moved = [&](const void *p) {
    const uintptr_t a = (uintptr_t)p;
    return a >= lo && a < hi ? (void *)((uintptr_t)new_base + (a - lo)) : (void *)p;
  };
  // the ops with their operands moved; nothing of the graph changes until this has been checked
  std::vector<pccl_op_desc> next = G->descs;  // (dependency lists stay where they are, in deps_store)
  for (size_t i = 0; i < next.size(); ++i) {
    pccl_op_desc &o = next[i];
    // a signal word moves like an operand; it is 4 bytes whatever the op's dtype field says
    const bool is_signal = o.primitive == PCCL_NOTIFY || o.primitive == PCCL_GET_NOTIFIED;
    const uintptr_t es = is_signal ? 4 : (uintptr_t)elem_bytes(o.dtype);
    for (int k = 0; k < o.n_in + o.n_out; ++k) {
      void *p = moved(k < o.n_in ? o.ins[k] : o.outs[k - o.n_in]);
      if ((uintptr_t)p % es)
        return fail(PCCL_ERR_MISALIGNED, "graph_rebind: op %zu operand %d would not be %d-byte aligned", i, k, (int)es);
      if (k < o.n_in) o.ins[k] = p;
      else o.outs[k - o.n_in] = p;
    }
  }
  if (G->as_launches) {
    // The plan was made for the old addresses (which copies fold into their producers, which ops
    // continue each other); it is made again for the new ones.  Nothing on the device changes.
    std::vector<pccl_op_desc> plan;
    if (!plan_launches(next, &plan))
      return fail(PCCL_ERR_UNSUPPORTED, "graph_rebind: with these addresses the graph no longer runs as plain launches; create it again");
    for (const pccl_op_desc &o : plan) {
      const int rc = check_launch(o);
      if (rc != PCCL_OK) return rc;
    }
    G->descs.swap(next);
    G->launches.swap(plan);
    return PCCL_OK;
  }
  // Which dependencies may be met part by part depends on which operands share addresses
  // (an output tensor that now is the input tensor, say).  If that changed, the arena's
  // contents are built again from the moved ops, in place (its layout does not depend on
  // addresses, and launches recorded by stream capture point at it); earlier runs on `stream`
  // finish first.  Only a failed upload can leave the graph unusable.
  // ... and so does which ops run as chains behind each other, and how (plan_chains).
  const std::vector<pccl_op_desc> eff_next = effective_of(G, next);
  std::vector<LaunchChain> rows_next;
  int shape_next = 0;
  const std::vector<unsigned char> edges_after = classify_dependencies(eff_next, G->parts, G->topo, &G->part_eligible);
  if (edges_after != G->part_edge || plan_chains_of(G, eff_next, G->parts, edges_after, G->forward_capable ? G->kernel_elem_bytes : 0) != G->chain_words) {
    PCCL_HIP_CHECK(hipStreamSynchronize((hipStream_t)stream));
    Graph fresh;
    fresh.descs.swap(next);
    fresh.tile_bytes = G->tile_bytes;
    fresh.trace = G->trace;
    fresh.trace_on = G->trace_on;
    fresh.spin_limit = G->spin_limit;
    fresh.fixed_parts = G->parts;
    fresh.fixed_n_wg = G->n_wg;
    fresh.fixed_kernel = G->kernel;
    fresh.forward_capable = G->forward_capable;
    fresh.want_wide = G->wide;  // (a wide launch stays one, or the rebind is refused before anything changes)
    if (G->wide) fresh.fixed_chains = G;  // (... and runs as the same launch)
    fresh.wide_lds = G->wide_lds;
    fresh.wide_small = G->wide_small;
    char *old_dev = G->dev;
    // The run number goes on from where the DEVICE stands, not from the count of graph_run
    // calls: every replay of a recorded launch has moved the device's word on as well, and a
    // word set back would let the signal values that earlier replays left behind satisfy the
    // waits of the next run before its data exists.
    unsigned int run_word = G->runs + 1u;
    {
      const size_t off_hot = (size_t)((const char *)((const GraphControl *)G->image.data())->hot - G->dev);
      PCCL_HIP_CHECK(hipMemcpy(&run_word, G->dev + off_hot + sizeof(HotWord) * kHotRun, sizeof(run_word),
                               hipMemcpyDeviceToHost));
      // A run that gave up and that nobody has asked about yet: the new state would bury its abort
      // word.  Nothing is changed; pccl_hip_graph_status reports that run and restores the graph.
      unsigned int gave_up = 0;
      PCCL_HIP_CHECK(hipMemcpy(&gave_up, G->dev + off_hot + sizeof(HotWord) * kHotAbort, sizeof(gave_up),
                               hipMemcpyDeviceToHost));
      if (gave_up)
        return fail(PCCL_ERR_GRAPH, "graph_rebind: the graph's last run gave up and has not been reported yet; "
                                    "call pccl_hip_graph_status first (it restores the graph), then rebind");
    }
    const int rc = build_graph(&fresh, run_word, G->dev, G->arena_bytes);
    if (rc != PCCL_OK) return rc;
    G->runs = run_word - 1u;  // pccl_hip_graph_next_signal_base follows the device from here
    G->dev = fresh.dev;
    G->arena_bytes = fresh.arena_bytes;
    G->image.swap(fresh.image);
    G->payload_off = fresh.payload_off;
    G->chain_table_off = fresh.chain_table_off;
    G->total_tiles = fresh.total_tiles;
    G->all_tiles = fresh.all_tiles;
    G->n_wg = fresh.n_wg;
    G->wide_ok = fresh.wide_ok;
    G->chains_args = fresh.chains_args;  // (the same launch as before; the table's address is the arena's)
    G->chains_off = fresh.chains_off;
    G->device = fresh.device;
    G->kernel = fresh.kernel;
    G->descs.swap(fresh.descs);
    G->parts.swap(fresh.parts);
    G->topo.swap(fresh.topo);
    G->part_edge.swap(fresh.part_edge);
    G->part_eligible.swap(fresh.part_eligible);
    G->n_succ.swap(fresh.n_succ);
    G->order_touch.swap(fresh.order_touch);
    G->chain_words.swap(fresh.chain_words);
    G->eff.swap(fresh.eff);
    G->eff_deps.swap(fresh.eff_deps);
    G->fused_into.swap(fresh.fused_into);
    G->wait_of.swap(fresh.wait_of);
    G->notify_of.swap(fresh.notify_of);
    G->signal_cut.swap(fresh.signal_cut);
    G->user_dep_to_eff.swap(fresh.user_dep_to_eff);
    G->fuse_table_off = fresh.fuse_table_off;
    if (old_dev != G->dev) PCCL_HIP_CHECK(hipFree(old_dev));
    return PCCL_OK;
  }
  if (G->chains_launch && (!launch_chains_of(eff_next, G->chain_words, G->chains_dtype, G->chains_compute, &rows_next, &shape_next) ||
                           (int)rows_next.size() != G->chains_args.n_chains))
    return fail(PCCL_ERR_UNSUPPORTED, "graph_rebind: with these operands the graph no longer runs as the launch it was made for; create it again");
  G->descs.swap(next);
  for (size_t i = 0; i < G->eff.size(); ++i) {  // (the same ops: the dependency lists stay, the operands move)
    memcpy(G->eff[i].ins, eff_next[i].ins, sizeof(G->eff[i].ins));
    memcpy(G->eff[i].outs, eff_next[i].outs, sizeof(G->eff[i].outs));
  }
  char *payloads = G->image.data() + G->payload_off;
  for (int i = 0; i < G->n_ops; ++i) {
    pccl_op_payload *pl = (pccl_op_payload *)(payloads + kPayloadStride * (size_t)i);
    const int nc = pl->n_in_ + pl->n_out_;
    for (int k = 0; k < nc; ++k) pl->chunks_[k].addr_ = moved(pl->chunks_[k].addr_);
  }
  // ordered after earlier runs on `stream`; the source is pageable host memory,
  // so the call returns once the bytes are staged
  fill_chain_table(G->chain_words, G->n_ops, payloads, (ForwardStep *)(G->image.data() + G->chain_table_off));
  fill_fuse_table(G, G->eff, (SignalFuse *)(G->image.data() + G->fuse_table_off));
  PCCL_HIP_CHECK(hipMemcpyAsync(G->dev + G->payload_off, payloads,
                                G->fuse_table_off + sizeof(SignalFuse) * (size_t)G->n_ops - G->payload_off,
                                hipMemcpyHostToDevice, (hipStream_t)stream));
  if (G->chains_launch) {
    const LaunchChain *before = (const LaunchChain *)(G->image.data() + G->chains_off);
    for (size_t k = 0; k < rows_next.size(); ++k) rows_next[k].first_wg = before[k].first_wg;  // (the same ops of the same lengths)
    memcpy(G->image.data() + G->chains_off, rows_next.data(), sizeof(LaunchChain) * rows_next.size());
    PCCL_HIP_CHECK(hipMemcpyAsync(G->dev + G->chains_off, G->image.data() + G->chains_off, sizeof(LaunchChain) * rows_next.size(),
                                  hipMemcpyHostToDevice, (hipStream_t)stream));
  }
  return PCCL_OK;
}

int pccl_hip_graph_info(void *graph, void **device_layout, int *n_tiles, int *n_workgroups) {
  pccl_host::clear_error();
  Graph *G = (Graph *)graph;
  if (!G) return fail(PCCL_ERR_INVALID_ARG, "graph_info: graph is null");
  if (device_layout) *device_layout = G->dev;  // null for a graph that runs as plain launches
  if (n_tiles) *n_tiles = G->as_launches ? (int)G->launches.size() : G->total_tiles;
  if (n_workgroups) *n_workgroups = G->n_wg;  // 0 for a graph that runs as plain launches
  return PCCL_OK;
}

int pccl_hip_graph_launch_kind(void *graph, int *kind) {
  pccl_host::clear_error();
  Graph *G = (Graph *)graph;
  if (!G || !kind) return fail(PCCL_ERR_INVALID_ARG, "graph_launch_kind: null argument");
  *kind = G->as_launches ? 2 : G->chains_launch ? 3 : G->wide ? 1 : 0;
  return PCCL_OK;
}

int pccl_hip_classify_dependencies(const pccl_op_desc *ops, int n_ops, const int *parts, unsigned char *kinds) {
  pccl_host::clear_error();
  if (n_ops < 0 || (n_ops > 0 && (!ops || !parts))) return fail(PCCL_ERR_INVALID_ARG, "classify_dependencies: bad arguments");
  std::vector<pccl_op_desc> descs(ops, ops + n_ops);
  std::vector<int> part_counts(parts, parts + n_ops), indeg(n_ops, 0), topo;
  std::vector<std::vector<int>> succ(n_ops);
  size_t n_deps = 0;
  for (int i = 0; i < n_ops; ++i) {
    const pccl_op_desc &o = ops[i];
    if (o.n_deps < 0 || (o.n_deps > 0 && !o.deps)) return fail(PCCL_ERR_GRAPH, "op %d: bad dependency list", i);
    if (parts[i] < 1 || o.count < 0 || o.dtype >= PCCL_NUM_DTYPES || o.n_in > PCCL_MAX_INPUTS || o.n_out > PCCL_MAX_OUTPUTS)
      return fail(PCCL_ERR_INVALID_ARG, "op %d: bad part count, count, dtype or operand count", i);
    for (int d = 0; d < o.n_deps; ++d) {
      if (o.deps[d] < 0 || o.deps[d] >= n_ops || o.deps[d] == i) return fail(PCCL_ERR_GRAPH, "op %d: dependency %d is not another op", i, o.deps[d]);
      succ[o.deps[d]].push_back(i);
      ++indeg[i];
    }
    n_deps += (size_t)o.n_deps;
  }
  for (int i = 0; i < n_ops; ++i)
    if (!indeg[i]) topo.push_back(i);
  for (size_t k = 0; k < topo.size(); ++k)
    for (int v : succ[topo[k]])
      if (--indeg[v] == 0) topo.push_back(v);
  if ((int)topo.size() != n_ops) return fail(PCCL_ERR_GRAPH, "dependency graph has a cycle");
  const std::vector<unsigned char> flags = classify_dependencies(descs, part_counts, topo);
  if (n_deps && !kinds) return fail(PCCL_ERR_INVALID_ARG, "classify_dependencies: kinds is null");
  if (n_deps) memcpy(kinds, flags.data(), n_deps);
  return PCCL_OK;
}

int pccl_hip_plan_chains(const pccl_op_desc *ops, int n_ops, const int *parts, int forward_elem_bytes, int *words) {
  pccl_host::clear_error();
  if (n_ops < 0 || (n_ops > 0 && (!ops || !parts || !words))) return fail(PCCL_ERR_INVALID_ARG, "plan_chains: bad arguments");
  std::vector<unsigned char> kinds;
  {
    size_t n_deps = 0;
    for (int i = 0; i < n_ops; ++i) n_deps += (size_t)std::max(ops[i].n_deps, 0);
    kinds.assign(std::max<size_t>(n_deps, 1), 0);
  }
  const int rc = pccl_hip_classify_dependencies(ops, n_ops, parts, kinds.data());  // checks the ops as well
  if (rc != PCCL_OK) return rc;
  std::vector<pccl_op_desc> descs(ops, ops + n_ops);
  std::vector<int> part_counts(parts, parts + n_ops), n_succ(n_ops, 0);
  for (int i = 0; i < n_ops; ++i)
    for (int d = 0; d < ops[i].n_deps; ++d) ++n_succ[ops[i].deps[d]];
  const std::vector<unsigned char> untouched(n_ops, 0);
  const std::vector<int> plan = plan_chains(descs, part_counts, kinds, n_succ, untouched, forward_elem_bytes);
  if (n_ops) memcpy(words, plan.data(), sizeof(int) * (size_t)kChainWords * (size_t)n_ops);
  return PCCL_OK;
}

int pccl_hip_plan_signals(const pccl_op_desc *ops, int n_ops, int *carrier, int *parts) {
  pccl_host::clear_error();
  if (n_ops < 0 || (n_ops > 0 && (!ops || !carrier))) return fail(PCCL_ERR_INVALID_ARG, "plan_signals: bad arguments");
  for (int i = 0; i < n_ops; ++i) {
    const pccl_op_desc &o = ops[i];
    if (o.primitive > PCCL_GET_NOTIFIED) return fail(PCCL_ERR_UNSUPPORTED, "op %d: unknown primitive code %d", i, o.primitive);
    if (o.n_deps < 0 || (o.n_deps > 0 && !o.deps)) return fail(PCCL_ERR_GRAPH, "op %d: bad dependency list", i);
    for (int d = 0; d < o.n_deps; ++d)
      if (o.deps[d] < 0 || o.deps[d] >= n_ops || o.deps[d] == i) return fail(PCCL_ERR_GRAPH, "op %d: dependency %d is not another op", i, o.deps[d]);
  }
  Graph G;
  G.descs.assign(ops, ops + n_ops);
  fuse_signals(&G);
  for (int i = 0; i < n_ops; ++i) carrier[i] = G.fused_into[i];
  if (parts)
    for (int i = 0; i < n_ops; ++i)
      parts[i] = G.fused_into[i] >= 0 ? (ops[i].signal_parts >= 2 ? (int)ops[i].signal_parts : 0) : G.signal_cut[i];
  return PCCL_OK;
}

int pccl_hip_graph_dependency_kinds(void *graph, unsigned char *kinds, long capacity, long *n_deps) {
  pccl_host::clear_error();
  Graph *G = (Graph *)graph;
  if (!G || !n_deps) return fail(PCCL_ERR_INVALID_ARG, "graph_dependency_kinds: null argument");
  if (capacity < 0 || (capacity > 0 && !kinds)) return fail(PCCL_ERR_INVALID_ARG, "graph_dependency_kinds: bad buffer");
  std::lock_guard<std::mutex> lock(G->mu);
  // per dependency as the caller listed them; one that a carried signal op took part in is met by the
  // data op's own waiting and reports whole-op; a graph run as launches: stream order, whole-op
  *n_deps = (long)G->deps_store.size();
  const long n = std::min<long>(capacity, *n_deps);
  for (long k = 0; k < n; ++k) {
    const long place = (!G->as_launches && (size_t)k < G->user_dep_to_eff.size()) ? G->user_dep_to_eff[(size_t)k] : -1;
    kinds[k] = place >= 0 ? G->part_edge[(size_t)place] : 0;
  }
  return PCCL_OK;
}

int pccl_hip_graph_next_signal_base(void *graph, unsigned int *base) {
  pccl_host::clear_error();
  Graph *G = (Graph *)graph;
  if (!G || !base) return fail(PCCL_ERR_INVALID_ARG, "graph_next_signal_base: null argument");
  std::lock_guard<std::mutex> lock(G->mu);
  *base = (G->runs + 1u) << 16;
  return PCCL_OK;
}

int pccl_hip_graph_set_spin_limit(void *graph, unsigned int microseconds) {
  pccl_host::clear_error();
  Graph *G = (Graph *)graph;
  if (!G) return fail(PCCL_ERR_INVALID_ARG, "graph_set_spin_limit: graph is null");
  const unsigned int limit = std::max(microseconds, 64u);  // (the kernel looks at the clock every 64 polls anyway)
  std::lock_guard<std::mutex> lock(G->mu);
  G->spin_limit = limit;
  if (G->as_launches) return PCCL_OK;  // nothing waits inside plain launches
  ((GraphControl *)G->image.data())->spin_limit = limit;
  PCCL_HIP_CHECK(hipMemcpy(G->dev + offsetof(GraphControl, spin_limit), &limit, sizeof(limit), hipMemcpyHostToDevice));
  return PCCL_OK;
}

int pccl_hip_graph_run_static(const pccl_op_desc *ops, int n_ops, long tile_bytes, void *stream,
                              unsigned int *completed, unsigned int *total) {
  pccl_host::clear_error();
  if (n_ops < 0 || (n_ops > 0 && !ops)) return fail(PCCL_ERR_INVALID_ARG, "graph_run_static: bad op array");
  if (tile_bytes < 0) return fail(PCCL_ERR_INVALID_ARG, "graph_run_static: tile_bytes %ld < 0", tile_bytes);
  if (completed) *completed = 0;
  if (total) *total = (unsigned int)n_ops;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return fail(PCCL_ERR_NO_DEVICE, "no current device");
  std::lock_guard<std::mutex> lock(g_static_mutex);
  if (dev < 0 || dev >= kMaxStaticDevices) return fail(PCCL_ERR_UNSUPPORTED, "graph_run_static: device index %d", dev);
  StaticArena &S = g_static[dev];
  if (!S.ptr) {
    // set-up, once per device, with that device current: where this device keeps its copy of the array
    void *p = nullptr;
    PCCL_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(g_static_arena)));
    S.ptr = (char *)p;
    S.graph = new Graph();
  }
  // own copy of the ops and their dependency lists
  size_t n_deps = 0;
  for (int i = 0; i < n_ops; ++i) {
    if (ops[i].n_deps < 0 || (ops[i].n_deps > 0 && !ops[i].deps)) return fail(PCCL_ERR_GRAPH, "op %d: bad dependency list", i);
    n_deps += (size_t)ops[i].n_deps;
  }
  std::vector<int> &deps = S.deps;
  deps.clear();
  deps.reserve(n_deps);
  for (int i = 0; i < n_ops; ++i) deps.insert(deps.end(), ops[i].deps, ops[i].deps + ops[i].n_deps);
  Graph *G = S.graph;
  // Every call on this GPU shares the one array, so the previous call's run ends first, whatever stream
  // it went to and whether or not this call brings the same ops: two drains on the one state would race,
  // and a new upload would pull the state from under a running one.  With the run over, its abort word
  // says whether a wait inside it gave up.  A caller that passed no counters has not heard of that; it
  // hears now, nothing is launched on the abandoned state (every workgroup would leave at once and the
  // outputs would stay as they are), and the call after this one uploads the state afresh.
  if (S.used) PCCL_HIP_CHECK(hipStreamSynchronize(S.last_stream));
  if (S.valid && S.launched) {
    const size_t off_hot = (size_t)((const char *)((const GraphControl *)G->image.data())->hot - G->dev);
    unsigned int gave_up = 0;
    PCCL_HIP_CHECK(hipMemcpy(&gave_up, G->dev + off_hot + sizeof(HotWord) * kHotAbort, sizeof(gave_up), hipMemcpyDeviceToHost));
    if (gave_up) {
      S.valid = false;
      S.launched = false;
      return fail(PCCL_ERR_GRAPH, "graph_run_static: the previous run on this GPU gave up (an op's dependencies or a signal "
                                  "were not satisfied within the spin limit); nothing was launched, the next call uploads fresh state");
    }
  }
  auto same_ops = [&] {
    if (!S.valid || (int)G->descs.size() != n_ops || G->tile_bytes != tile_bytes || G->deps_store != deps ||
        G->spin_limit != default_spin_limit())
      return false;
    for (int i = 0; i < n_ops; ++i) {
      const pccl_op_desc &a = G->descs[i], &b = ops[i];
      if (a.op_uid != b.op_uid || a.primitive != b.primitive || a.dtype != b.dtype || a.compute != b.compute ||
          a.n_in != b.n_in || a.n_out != b.n_out || a.count != b.count || a.n_deps != b.n_deps || a.signal_parts != b.signal_parts ||
          memcmp(a.ins, b.ins, sizeof(void *) * b.n_in) || memcmp(a.outs, b.outs, sizeof(void *) * b.n_out))
        return false;
    }
    return true;
  };
  if (!same_ops()) {
    S.valid = false;
    S.launched = false;
    G->tile_bytes = tile_bytes;
    G->spin_limit = default_spin_limit();
    G->descs.assign(ops, ops + n_ops);
    G->deps_store.swap(deps);
    for (int i = 0, at = 0; i < n_ops; at += ops[i].n_deps, ++i) G->descs[i].deps = G->deps_store.data() + at;
    const FixedArena fixed{S.ptr, kStaticArenaBytes, (hipStream_t)stream};
    const int rc = build_graph(G, S.runs + 1u, nullptr, 0, &fixed);  // the whole image, zeros included, goes up: nothing of the last call's state survives
    if (rc != PCCL_OK) return rc;
    S.valid = true;
  }
  S.used = true;
  S.last_stream = (hipStream_t)stream;
  if (G->total_tiles > 0) {
    GraphControl control;
    memcpy(&control, G->image.data(), sizeof(control));
    hipLaunchKernelGGL(G->kernel, dim3((unsigned)G->n_wg), dim3(kBlock), 0, (hipStream_t)stream, control);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(PCCL_ERR_HIP, "graph_run_static launch failed: %s", hipGetErrorString(e));
    ++S.runs;
    S.launched = true;
  }
  if (!completed && !total) return PCCL_OK;
  PCCL_HIP_CHECK(hipStreamSynchronize((hipStream_t)stream));
  if (G->total_tiles == 0) return PCCL_OK;
  const size_t off_hot = (size_t)((const char *)((const GraphControl *)G->image.data())->hot - G->dev);
  HotWord hot[kHotWords];
  PCCL_HIP_CHECK(hipMemcpy(hot, G->dev + off_hot, sizeof(hot), hipMemcpyDeviceToHost));
  if (completed) *completed = hot[kHotCompleted].value;
  if (total) *total = hot[kHotTotal].value;
  if (hot[kHotAbort].value) {
    S.valid = false;  // the next call uploads a fresh image
    S.launched = false;
    return fail(PCCL_ERR_GRAPH, "drain gave up: an op's dependencies were not satisfied within the spin limit "
                                "(%u of %u ops had completed)", hot[kHotCompleted].value, hot[kHotTotal].value);
  }
  return PCCL_OK;
}

int pccl_hip_graph_destroy(void *graph) {
  pccl_host::clear_error();
  Graph *G = (Graph *)graph;
  if (!G) return PCCL_OK;
  hipError_t e = G->dev ? hipFree(G->dev) : hipSuccess;
  if (G->trace) {
    const hipError_t e2 = hipFree(G->trace);
    if (e == hipSuccess) e = e2;
  }
  delete G;
  if (e != hipSuccess) return fail(PCCL_ERR_HIP, "hipFree of the op graph: %s", hipGetErrorString(e));
  return PCCL_OK;
}

}  // extern "C"
