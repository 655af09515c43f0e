// schedule.h -- a compiled collective: the op list Engine::regOp(name, filepath)
// loads, its on-disk text format, and native generators.
//
// The reference passes a file path to regOp (include/engine.h:18) but defines
// neither the format nor a producer (csrc/engine.cc:102-104 is empty,
// pccl/lang/operator.py and example/collective/allreduce.py are empty files).
// An op record carries what a PrimitiveOp of pccl/lang/chunk.py:46-55 carries:
// kind, id (= position), source / target chunks as (buffer, device, element
// offset), element count, dependencies.
//
// File format, one token stream, '#' starts a comment line:
//   pccl-schedule 1
//   name <word>
//   dtype <f32|i32|bf16|f16>
//   compute <sum|prod|min|max>
//   devices <W>
//   elems_per_device <N>          elements of every device's "in" and "out" region
//   ops <n>
//   op <id> <COPY|REDUCE> <count> deps <k> <id>*k  src <s> (<buffer> <device> <offset>)*s
//                                                  dst <d> (<buffer> <device> <offset>)*d
//   op <id> <NOTIFY|GET_NOTIFIED> <value> deps <k> <id>*k slot <index>
// A signal op names one of the device workspace's int signal slots (csrc/engine.cc:16-18:
// 256 slots behind the 256 MiB workspace) and a value in [0, 65535]; NOTIFY publishes the
// value once its dependencies are complete, GET_NOTIFIED completes when the slot has
// reached it (pccl/lang/chunk.py:9-10).
// Version 2 ("pccl-schedule 2"; version 1 files load as before) differs in one thing: a signal
// op line ends in "parts <K>", and with K >= 2 the signal is K consecutive slots from <index>,
// slot p standing for part p of the data op it follows (NOTIFY) or precedes (GET_NOTIFIED), the
// op cut into K parts (part p = elements [p * per, (p + 1) * per), per = ceil(count / K) rounded
// up to 64).  The executor then lets the consumer start on part p as soon as the producer has
// finished its part p (pccl_hip.h, pccl_op_desc::signal_parts).
// Buffers: "in" and "out" are the tensors given to exeOp, laid out as W consecutive
// per-device regions of elems_per_device elements; "ws" is the device workspace.
#pragma once

#include <string>
#include <vector>

namespace engine_c {

struct ScheduleOperand {
  std::string buffer;  // "in", "out" or "ws"
  int device = 0;
  long offset = 0;     // elements, inside the device's region
};

struct ScheduleOp {
  enum Kind { COPY, REDUCE, NOTIFY, GET_NOTIFIED };
  Kind kind = COPY;
  bool reduce = false;  // kind == REDUCE (kept in step with kind by the parser and generators)
  bool isSignal() const { return kind == NOTIFY || kind == GET_NOTIFIED; }
  int slot = 0;         // signal ops: index of the signal slot; count is the value
  int parts = 1;        // signal ops: slots the signal takes, one per part of the data (format version 2)
  long count = 0;
  std::vector<int> deps;
  std::vector<ScheduleOperand> srcs;
  std::vector<ScheduleOperand> dsts;
};

struct Schedule {
  std::string name;
  std::string dtype = "bf16";
  std::string compute = "sum";
  int devices = 1;
  long elems_per_device = 0;
  std::vector<ScheduleOp> ops;

  int elemBytes() const;
  // Structural checks: operand ranges, dependency ids, acyclicity.  Throws std::runtime_error.
  void validate() const;
  // Op ids in the order DirectedGraph.topological_sort of pccl/lang/utils/graph.py:94-112
  // produces for this DAG (reverse DFS post-order, nodes in id order, successors in
  // edge-insertion order).
  std::vector<int> topologicalOrder() const;

  std::string serialize() const;
  static Schedule parse(const std::string &text);
  static Schedule load(const std::string &path);
  void save(const std::string &path) const;
};

// Appends an out-of-place ring all-reduce over `devices` virtual ranks, `chunk_elems`
// elements per chunk, regions starting at element `base`; returns the new base.
long appendRingAllReduce(Schedule &s, long chunk_elems, long base);

// Direct ("NVLS-style") all-reduce: device d reduces slice d of all W inputs in one
// W-input op and writes it to every device's output (W outputs), W ops, no dependencies.
long appendDirectAllReduce(Schedule &s, long slice_elems, long base);

// The two halves of the ring on their own.  Reduce-scatter: after W-1 steps device r holds the
// fold of chunk (r+1) mod W in its "out".  All-gather: device r contributes chunk r of its "in";
// afterwards every "out" holds all W chunks.
long appendRingReduceScatter(Schedule &s, long chunk_elems, long base);
long appendRingAllGather(Schedule &s, long chunk_elems, long base);

// Broadcast of `elems` elements of device `root`'s "in" into every device's "out": one COPY
// with W destinations (W <= 8).
long appendBroadcast(Schedule &s, long elems, int root, long base);

// All-to-all: device r's "in" chunk d goes to device d's "out" chunk r; W*W independent copies.
long appendAllToAll(Schedule &s, long chunk_elems, long base);

// The small-message program: n_slices ring all-reduces with log-uniform chunk sizes in
// [lo_bytes, hi_bytes] plus n_extra independent copies; seed selects the sizes.
Schedule makeSmallMessageSchedule(int devices, int n_slices, int n_extra, unsigned long seed,
                                  long lo_bytes, long hi_bytes, const std::string &dtype);

}  // namespace engine_c
