/*
 * pccl_hip.h -- C ABI of the MI355X (gfx950) reduce-copy plugin, libpccl_hip.so.
 *
 * This is the boundary the reference's host code binds for its local
 * reduce-copy / copy path.  In the reference that path is declared but empty:
 *   - include/plugins/cuda_executor/executor.h   (0 bytes; device executor)
 *   - include/plugins/cpu_executor/executor.h    (0 bytes; CPU executor)
 *   - csrc/engine.cc:102-104 Engine::regOp, include/engine.h:19 Engine::exeOp
 * so each entry point below cites the reference declaration whose role it
 * fills.  Plain pointers and sizes only; no C++ or torch types; no exception
 * crosses this boundary.  Every function returns PCCL_OK (0) or a negative
 * PCCL_ERR_* code; pccl_hip_last_error() gives the text for the calling thread.
 */
#ifndef PCCL_HIP_H
#define PCCL_HIP_H

#include "pccl_op_layout.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ---- return codes -------------------------------------------------------- */
#define PCCL_OK 0
#define PCCL_ERR_INVALID_ARG (-1) /* null pointer, count < 0, n_in/n_out out of range ...  */
#define PCCL_ERR_UNSUPPORTED (-2) /* unknown dtype / compute / primitive code               */
#define PCCL_ERR_HIP (-3)         /* a HIP runtime call failed; text in last_error          */
#define PCCL_ERR_NO_DEVICE (-4)   /* no gfx950 device visible                               */
#define PCCL_ERR_NOMEM (-5)       /* device allocation failed                               */
#define PCCL_ERR_MISALIGNED (-6)  /* operand address not a multiple of its element size     */
#define PCCL_ERR_GRAPH (-7)       /* op graph malformed: cycle, bad uid, too many edges ... */

/* ---- fixed codes used on the wire ---------------------------------------- */
/* The host layer maps TypeRegistry ids (include/base/registry.h:12-43, ids are
 * handed out at run time from one shared counter) onto these stable codes. */
enum pccl_dtype {   /* element types with 16-byte packs in                         */
  PCCL_F32 = 0,     /* include/plugins/cuda_executor/utils/vector_datatype.h:66    */
  PCCL_I32 = 1,     /* :64                                                         */
  PCCL_BF16 = 2,    /* :71 (bf16x8)                                                */
  PCCL_F16 = 3,     /* :70 (f16x8)                                                 */
  PCCL_F8E4M3 = 4,  /* :75-77 (fp8_e4m3 packs): OCP E4M3FN, 16 per 16-byte pack     */
  PCCL_F8E5M2 = 5,  /* :78-80 (fp8_e5m2 packs): OCP E5M2                            */
  PCCL_F64 = 6,     /* the f64 of multimemStore (utils/multimem.h:61-102); 2 per pack */
  PCCL_U32 = 7      /* :66-68 (u32 packs) and multimem.h's u32 add; min / max unsigned */
};
#define PCCL_NUM_DTYPES 8

/* Element size in bytes of a dtype code (the scalar types of vector_datatype.h:55-80),
 * 0 for an unknown code. */
int pccl_hip_dtype_bytes(int dtype);
enum pccl_compute { /* multimem.h:12-59 only has .add; min/max/prod complete the   */
  PCCL_SUM = 0,     /* set of ComputeType names the registry is meant to hold      */
  PCCL_PROD = 1,
  PCCL_MIN = 2,
  PCCL_MAX = 3
};
enum pccl_primitive { /* PrimitiveOpType, pccl/lang/chunk.py:6-10 */
  PCCL_COPY = 0,
  PCCL_REDUCE = 1,
  PCCL_NOTIFY = 2,
  PCCL_GET_NOTIFIED = 3
};

#define PCCL_MAX_INPUTS 8
#define PCCL_MAX_OUTPUTS 8

/* ---- device + allocator --------------------------------------------------- */

/* Number of usable devices.  Role: CudaDevice::allocatorAvailable,
 * csrc/plugins/cuda_executor/device.cc:53-57 (cudaGetDeviceCount > 0). */
int pccl_hip_device_count(int *n);

/* Compute units and HBM bytes of the current device (launch sizing and
 * reporting; the reference has no counterpart because it has no launches). */
int pccl_hip_device_info(int *compute_units, long *hbm_bytes, char *name, int name_len);

/* The id under which the host's TypeRegistry registered this executor (registerExecutorType,
 * include/base/registry.h:37; ids come from one run-time counter, :79).  The plugin writes it into
 * RingBuffer::producer_ / consumer_ (include/base/operator.h:8-9) and
 * OperationLayoutHeader::executor_type_ (:24) of every graph created afterwards; a caller of the bare
 * C ABI that never sets it gets 0 there.  0..255. */
int pccl_hip_set_executor_id(int id);

/* Device memory, tracked until freed: one hipMalloc per call, the size rounded up to 2 MiB, in a
 * pointer-keyed map under a mutex.  nbytes <= 0 yields PCCL_ERR_INVALID_ARG and *p == NULL.
 * Role: CudaDevice::allocate / deallocate, csrc/plugins/cuda_executor/device.cc:59-144 (2 MiB
 * granularity :60,70; nullptr for nbytes <= 0 :61; pointer-keyed bookkeeping :121-144).
 * pccl_hip_free waits, like hipFree, for the work that may still use the memory; called while the
 * thread records a stream capture it fails with PCCL_ERR_HIP and the buffer stays allocated. */
int pccl_hip_alloc(void **p, long nbytes);
int pccl_hip_free(void *p);

/* ---- the hot path: one reduce-copy ---------------------------------------- */

/* out[j][i] = cvt(fold_op(up(in[0][i]) ... up(in[n_in-1][i]))) for j < n_out,
 * i < count.  Strict left fold in input order; float accumulator for
 * f32/bf16/f16/f8 with one round-to-nearest-even at the end (f8: saturating to the
 * largest finite value); uint32 wraparound for i32; n_in == 1 copies bytes.  Any element-aligned addresses; an output
 * may be the same buffer as an input (in place), other overlaps are undefined.
 * One kernel launch on `stream` (a hipStream_t; NULL = the default stream);
 * returns without waiting.
 * Role: the N-pointer form of multimem_ld_reduce + multimemStore,
 * include/plugins/cuda_executor/utils/multimem.h:12-102, over operands
 * described like ChunkMeta, include/base/chunk.h:10-14. */
int pccl_hip_reduce_copy(int dtype, int compute, const void *const *ins, int n_in,
                         void *const *outs, int n_out, long count, void *stream);

/* Folds ONE input into each of n_out destinations, reading the input once:
 *   outs[j][i] = cvt(op(up(outs[j][i]), up(in[i])))      (destination first, then the value).
 * The destinations must be distinct buffers that nothing else writes during the launch.
 * Role: multimemStoreReduce, include/plugins/cuda_executor/utils/multimem.h:104-127
 * (multimem.red.add of one pack into every peer's copy). */
int pccl_hip_accumulate(int dtype, int compute, const void *in, void *const *outs, int n_out, long count,
                        void *stream);

/* Launch-shape overrides for tuning runs: workgroups per compute unit
 * (0 = built-in choice) and cache treatment (-1 = built-in choice, 0 = cacheable,
 * 1 = non-temporal loads and stores, 2 = non-temporal loads and write-through stores). */
int pccl_hip_set_tuning(int workgroups_per_cu, int cache_treatment);

/* pccl_hip_reduce_copy and pccl_hip_accumulate launch one workgroup per 4 KiB of every operand, and a
 * launch holds at most 2^24 - 1 of them (just under 64 GiB per operand): longer operands run as
 * several launches over consecutive slices of `bytes` each (a multiple of 4096, at most and by default
 * 32 GiB; 0 = the default).  Smaller values only serve tests of that path. */
int pccl_hip_set_slice_bytes(long bytes);

/* Occupancy override for tuning runs: bytes of (unused) dynamic LDS requested per
 * workgroup, which caps the workgroups resident on a compute unit at
 * floor(160 KiB / lds_bytes); -1 = built-in choice, 0 = no cap. */
int pccl_hip_set_occupancy_lds(int lds_bytes);

/* Kernel-shape override for tuning runs: -1 = built-in choice, 0 = the lean one-pack-per-lane
 * kernel wherever it applies, 1 or 4 = packs per lane of the general kernel. */
int pccl_hip_set_unroll(int unroll);

/* Walk override for tuning runs: which 4 KiB chunk of the streams workgroup k of a direct launch takes.
 * 0 = chunk k; 1 = bits 5-7 of k XORed into its low three bits wherever the launch has one workgroup
 * per chunk, so that the workgroups in flight on one XCD read from all 8 HBM channel groups whatever the
 * operands' addresses are; -1 = built-in choice (rotated for operands beyond the Infinity Cache). */
int pccl_hip_set_rotation(int rotate);

/* ---- the op-batching path: a DAG of ops drained by one persistent kernel -- */

/* One IR operation as the host hands it over: the C++ payload level of
 * PrimitiveOp (pccl/lang/chunk.py:46-55): op kind, operands, dependencies.
 * Signal ops (chunk.py:9-10; signal words like the int slots of csrc/engine.cc:16-18):
 *   NOTIFY        n_in 0, n_out 1: outs[0] = address of a 32-bit signal word, count =
 *                 value (0..65535); once its dependencies are complete it stores
 *                 signal_base + value to the word (system scope);
 *   GET_NOTIFIED  n_in 1, n_out 0: ins[0] = signal word, count = value; it completes
 *                 when (int)(word - (signal_base + value)) >= 0 (bounded wait).
 * signal_base = run number << 16 (pccl_hip_graph_next_signal_base), so a word left over
 * from an earlier run never satisfies a wait of a later one.
 * Signals per part (signal_parts = K >= 2; 0 and 1 mean the one word above): the signal is K consecutive
 * 32-bit words, word p standing for part p of the data it announces, the data cut into K parts by the
 * rule that both sides know (part p = elements [p * per, min((p + 1) * per, count)), per =
 * ceil(count / K) rounded up to 64).  A NOTIFY whose only dependency is one COPY / REDUCE makes the
 * executor cut that op into exactly K parts, and whoever completes part p stores word p; a GET_NOTIFIED
 * that one COPY / REDUCE alone depends on makes that op K parts, and its part p polls word p only.  So a
 * consumer starts on the first part while the producer is still working on the others: a ring whose
 * ranks are linked by such pairs streams instead of stopping at every step.  (An op that would carry
 * signals of two different K carries the first; a per-part signal op that stands alone stores, or waits
 * for, all K words.)  Both ends of a pair must name the same K. */
typedef struct pccl_op_desc {
  int op_uid;                          /* dense 0..n_ops-1, chunk.py:82-83           */
  unsigned char primitive;             /* enum pccl_primitive                         */
  unsigned char dtype;                 /* enum pccl_dtype                             */
  unsigned char compute;               /* enum pccl_compute                           */
  unsigned char n_in;                  /* 1..8                                        */
  unsigned char n_out;                 /* 1..8                                        */
  unsigned char reserved;
  unsigned short signal_parts;         /* NOTIFY / GET_NOTIFIED: words of the signal (see above); else 0 */
  const void *ins[PCCL_MAX_INPUTS];
  void *outs[PCCL_MAX_OUTPUTS];
  long count;                          /* elements per operand                        */
  int n_deps;                          /* PrimitiveOp.dependencies, chunk.py:54       */
  const int *deps;                     /* op_uids that must complete first            */
} pccl_op_desc;

/* Builds the device-resident GraphBufferLayout (include/base/operator.h:31-38):
 * one OperationLayoutHeader per op (:19-29) with payload and successor list,
 * one ready queue (RingBuffer, :7-17).  Role: Engine::regOp,
 * csrc/engine.cc:102-104.  tile_bytes = bytes of output one workgroup handles
 * per queue entry; it fixes required_executors_.  0 = built-in choice: per dependency
 * level, 16 KiB x (bytes the level writes / 8 MiB)^(2/3), within 8 KiB to 128 KiB per part.
 * PCCL_HIP_TILE_AUTO = the executor's choice of HOW to run the graph as well (what Engine::exeOp
 * uses, whose caller cannot name an entry point): a graph that, after folding copies into the op that
 * produced their input and joining ops that continue each other, is at most two ops, or at most four
 * independent ops of 128 MiB of traffic or more each, runs as that many pccl_hip_reduce_copy launches
 * in dependency order (one op of 256 MiB per operand: 6.8 TB/s against 5.4 through the queue; the
 * one-exchange all-reduce over 8 ranks: one 8 -> 8 launch); every other graph goes to the queue with
 * the built-in part sizes.  For such a graph graph_status reports all ops complete once the stream has
 * drained, graph_info a null layout, graph_trace PCCL_ERR_UNSUPPORTED; a launch recorded by stream
 * capture keeps the addresses it was recorded with, whatever graph_rebind does later.
 * PCCL_HIP_PLAN_LAUNCHES=0 sends everything to the queue.
 * Chains: an op that depends on one op alone, which nothing else depends on and which is cut like
 * it, queues no entries of its own; the workgroup that has run part p of its predecessor goes on
 * with its part p (and keeps the value in registers where the op takes the predecessor's output 0
 * as one of at most two inputs; an output that a later op of the same such chain writes again at the
 * same address is then not stored by the earlier op: nothing could read it).  A level of the graph whose entries start such chains is cut by
 * the built-in choice into the smallest parts (from 8 KiB) with which its entries fit the resident
 * workgroups once.  In a chain that does not run in one pass, a COPY whose input is output 0 of the op before it is not run at
 * all: that op stores the copy's outputs as further outputs of its own (a slice folded 8 -> 1 and then copied 1 -> 7 is stored
 * as 8 -> 8), provided they fit one op and overlap none of its operands at another address; PCCL_HIP_FOLD_COPIES=0 runs it.
 * Results, graph_status and graph_rebind are as without chains;
 * graph_info's n_tiles and the timeline count the entries that are queued.  PCCL_HIP_CHAINS=0
 * switches chains off.
 * Signal ops that stand alone beside one data op ride on it: a NOTIFY whose only dependency is a
 * COPY / REDUCE is stored by whoever completes that op, and a GET_NOTIFIED that one COPY / REDUCE
 * alone depends on is polled by every part of that op (which takes over its dependencies); neither
 * queues an entry, both count as complete with the data op.  In the device image the successor list
 * of an op that carries a NOTIFY ends in -1 (next_op_uids_head_, num_next_ops_ counts it).
 * PCCL_HIP_FUSE_SIGNALS=0 keeps every signal op an op of its own.
 * The wide launch: with tile_bytes 0 (or PCCL_HIP_TILE_AUTO), a graph none of whose queue entries waits for
 * another entry or has to do with a signal word (independent ops; chains, whose later ops run behind the first
 * in the same workgroup) is cut into parts of 8 to 32 KiB and run by one short-lived workgroup per entry, as many
 * workgroups as entries, instead of the persistent drain: nothing is handed from workgroup to workgroup, so no
 * ticket is drawn and no part counted, and the hardware dispatcher balances the compute units (ring all-reduce
 * over 8 resident ranks x 1 / 8 / 32 / 64 MiB 16.4 / 30 / 92.5 / 227 -> 9.6 / 21.8 / 84.5 / 200 us, one 64 KiB op
 * 9.7 -> 6.5 us; entries outside one-pass chains are cut into 32 KiB parts once they move 192 MiB or more).
 * The device arena, graph_info, graph_trace and results are the same; graph_status reports every op complete
 * once the stream has drained (the launch's end is the graph's completion; *completed_operator on the device
 * is not written by such a launch); graph_rebind see there.  PCCL_HIP_WIDE=0: never.
 * Such a graph of at most 64 entries, each of which is one fold (one op of 2..8 inputs, with a COPY of its
 * result that it stores itself; or a chain that runs in one pass, takes at most 8 inputs in all and leaves
 * its final value in at most 8 outputs, every earlier output being overwritten by a later op of the chain:
 * the 14 ops of a ring all-reduce's chunk) over at least four streams, all ops of one element size, runs in
 * the shape of a direct launch instead: a workgroup per 4 KiB of every stream of a chain, the chains'
 * operands in a small table of the arena that all workgroups of a chain share (ring all-reduce over 8
 * resident ranks x 1 / 32 / 64 MiB 9.6 / 84.5 / 200 -> 7 / 80-83 / 172 us, direct all-reduce 8 x 32 MiB
 * 88 -> 79-81 us, within 3 % of one 8 -> 8 launch).  graph_info then reports workgroups for n_tiles, graph_trace records
 * one entry per workgroup.  A graph all of whose entries are copies to three or more outputs runs that way
 * from 48 MiB in all (all-gather or broadcast over 8 ranks x 128 MiB: 235 -> 167 us).  Other copies and folds
 * over fewer streams fit that launch too but are better off with the table (PCCL_HIP_CHAIN_LAUNCH=2 takes it
 * for them all the same).
 * PCCL_HIP_CHAIN_LAUNCH=0: the table-driven wide launch for these too. */
#define PCCL_HIP_TILE_AUTO (-1l)
int pccl_hip_graph_create(const pccl_op_desc *ops, int n_ops, long tile_bytes, void **graph);

/* Drains the whole DAG with ONE persistent-kernel launch on `stream`; returns
 * without waiting.  The graph re-arms itself, so it can be run again.  The calling thread's current
 * device must be the one the graph was created on (PCCL_ERR_INVALID_ARG otherwise).
 * Role: Engine::exeOp, include/engine.h:19. */
int pccl_hip_graph_run(void *graph, void *stream);

/* Waits for `stream`, then reports *completed_operator and *total_operator
 * (operator.h:32-33); after a successful run they are equal. */
int pccl_hip_graph_status(void *graph, void *stream, unsigned int *completed,
                          unsigned int *total);

/* Replaces operand addresses: every operand that lies in [old_base,
 * old_base+nbytes) moves to new_base + the same offset.  Lets exeOp bind a
 * new input / output tensor without rebuilding the graph: the new addresses are
 * uploaded behind earlier work on `stream`.  If the move changes which operands
 * share addresses (and with that which dependencies can be met part by part),
 * the call waits for `stream` and rewrites the graph's device arena in place
 * (launches recorded by stream capture stay valid).  A move that
 * would leave an operand unaligned for its element type returns
 * PCCL_ERR_MISALIGNED and changes nothing.  A graph that runs as a wide launch (see
 * pccl_hip_graph_create) cannot wait inside the launch: a move after which one of its entries
 * would have to wait for another (an op that no longer may run behind its predecessor part by
 * part, or chains that come out differently) returns PCCL_ERR_UNSUPPORTED and changes nothing;
 * create the graph again for such operands (Engine::exeOp does). */
int pccl_hip_graph_rebind(void *graph, const void *old_base, const void *new_base, long nbytes,
                          void *stream);

/* Per-entry timeline of the executor (no counterpart in the reference, whose headers
 * keep only the two progress counters of operator.h:32-33).  enable != 0 allocates 32 bytes
 * per queue entry once and makes the following runs record, per entry in queue order, four
 * 64-bit words: { op_uid | part << 32 | workgroup << 52, ticket drawn, dependencies met,
 * part complete }, times in ticks of the device's constant 100 MHz clock; each run
 * overwrites the last.  enable == 0 stops recording.  Not to be switched while a run is in
 * flight; a run recorded by stream capture keeps the setting it was recorded with.  read_trace waits for `stream`, copies up to `capacity` records (4 words each)
 * and reports the number of entries of the graph in *n_records. */
int pccl_hip_graph_trace(void *graph, int enable);
int pccl_hip_graph_read_trace(void *graph, void *stream, unsigned long long *records, long capacity,
                              long *n_records);

/* How the executor treats each dependency of the graph (no counterpart in the reference):
 * one byte per dependency, ops in uid order and each op's dependencies in list order;
 * 1 = met part by part (part p of the op waits only for part p of that predecessor, see
 * pccl_op_layout.h), 0 = the op waits for the whole predecessor (also reported for a dependency
 * from or on a signal op that rides on a data op: the data op does that waiting).  Copies up to
 * `capacity` bytes and reports the number of dependencies in *n_deps.  graph_rebind may change it. */
int pccl_hip_graph_dependency_kinds(void *graph, unsigned char *kinds, long capacity, long *n_deps);

/* The rule behind that, on its own: given the ops and the number of parts each is cut into
 * (part p of an op covers elements [p * per, min((p + 1) * per, count)) of every operand,
 * per = ceil(count / parts) rounded up to 64), writes one byte per dependency as above.
 * Touches no device; it exists so that the rule can be checked against every order of
 * execution it allows. */
int pccl_hip_classify_dependencies(const pccl_op_desc *ops, int n_ops, const int *parts, unsigned char *kinds);

/* Which ops the executor would run behind each other in one workgroup (chains, see graph_create), as
 * a host-only rule like the one above: given the ops, their part counts and the element size of the
 * graph's kernel instance (forward_elem_bytes; 0 = no chain may run in one pass), writes four ints per
 * op: the op that runs behind it (-1: none); for an op that starts a chain the number of ops in it
 * (else 1); for an op that starts a chain 1 if the chain runs in one pass with the value kept in
 * registers, for another op of such a chain the index of the input that is its predecessor's
 * output 0; and, for an op that starts a one-pass chain, the first of the chain's rows in the
 * executor's operand table.  In a chain that does not run in one pass the third int of a COPY that the op before it stores
 * (see graph_create) is 2.  Touches no device. */
int pccl_hip_plan_chains(const pccl_op_desc *ops, int n_ops, const int *parts, int forward_elem_bytes, int *words);

/* Which signal ops of a graph ride on data ops (no counterpart in the reference; touches no device):
 * carrier[i] = the COPY / REDUCE op that stores NOTIFY i when it completes, or whose parts poll
 * GET_NOTIFIED i before they start; -1 for every other op.  The rule is stated at
 * pccl_hip_graph_create; it looks at kinds, dependency lists and signal_parts only.
 * parts (may be NULL): for a signal op that is carried part by part (signal_parts >= 2, see pccl_op_desc)
 * its K; for the data op that carries such signals the K it is cut into; 0 for every other op. */
int pccl_hip_plan_signals(const pccl_op_desc *ops, int n_ops, int *carrier, int *parts);

/* Device address of the GraphBufferLayout and launch facts, for inspection: n_tiles = queue entries
 * (parts of the ops that queue entries; ops that run behind another op in a chain queue none), or the
 * number of launches for a graph that runs as plain launches; n_workgroups = width of the launch. */
int pccl_hip_graph_info(void *graph, void **device_layout, int *n_tiles, int *n_workgroups);

/* How the graph runs, for inspection: *kind = 0 the persistent drain, 1 a wide launch, 2 plain launches,
 * 3 a wide launch in the shape of a direct one (a few chains that are each one fold); see
 * pccl_hip_graph_create.  No counterpart in the reference. */
int pccl_hip_graph_launch_kind(void *graph, int *kind);

/* signal_base the NEXT pccl_hip_graph_run of this graph will use: a party outside the
 * graph that wants to satisfy a GET_NOTIFIED(value) stores *base + value to the word.
 * The run number itself lives on the device and moves on with every execution of the
 * drain kernel, so a pccl_hip_graph_run recorded into a HIP graph (stream capture) uses a
 * fresh base on every replay; this call counts pccl_hip_graph_run calls only, and a
 * caller that replays recorded runs adds 65536 per replay itself. */
int pccl_hip_graph_next_signal_base(void *graph, unsigned int *base);

/* Bounds every wait inside the drain kernel (for a dependency, for a signal word) to `microseconds`
 * by the device's constant 100 MHz clock (default 2,000,000: two seconds; the kernel looks at the clock
 * every 64 polls).  A caller whose graphs wait for peers, or run beside long kernels of other
 * streams, raises it.  When a wait gives up the kernel
 * raises its abort flag, every workgroup leaves, and pccl_hip_graph_status
 * returns PCCL_ERR_GRAPH after restoring the graph's pristine state.  Takes effect
 * with the next pccl_hip_graph_run (a run recorded by stream capture keeps the limit it
 * was recorded with). */
int pccl_hip_graph_set_spin_limit(void *graph, unsigned int microseconds);

/* pccl_hip_graph_create + pccl_hip_graph_run in one call that allocates NO device memory.  It has no
 * counterpart in the reference; it is for callers that cannot allocate: tight serving loops and harnesses
 * that forbid hipMalloc.  The graph's device state (headers, payloads, counters, ready queues: what
 * graph_create puts into a hipMalloc'ed arena) goes into a fixed array inside the library's code object,
 * of which every GPU holds one copy of PCCL_HIP_STATIC_ARENA_BYTES until the process ends.  (Host memory:
 * the library's own vectors, which stop growing once they have held the largest graph.)
 * All calls on one GPU share the one array, so a call first waits for the previous call's run to end,
 * whichever stream that went to, and looks at its abort word: if a wait inside that run gave up, this call
 * returns PCCL_ERR_GRAPH, launches nothing, and the call after it uploads the state afresh (a caller that
 * passes no counters learns of a failed run this way, one call late).  Then the call uploads the state
 * behind earlier work on `stream` and launches the drain kernel there; a call with the very same ops as
 * the last one on this GPU skips the upload (the state re-arms itself).  A graph that needs more than the
 * array holds (about 4,500 ops of three parts each) is refused with PCCL_ERR_NOMEM and nothing is launched.
 * completed / total both NULL: returns without waiting for the run it launched.  Otherwise waits for
 * `stream` and reports the graph's two progress counters (PCCL_ERR_GRAPH if the drain gave up; the next
 * call then uploads the state afresh).  Calls issued at the same time from several threads are
 * serialised by the library; work of the caller's own on other streams that touches the operands is the
 * caller's to order.  Not meant to be recorded by stream capture (the upload reads host memory and the
 * call waits for a stream).  Every graph goes through the persistent drain here (no wide launch). */
#define PCCL_HIP_STATIC_ARENA_BYTES (8u << 20)
int pccl_hip_graph_run_static(const pccl_op_desc *ops, int n_ops, long tile_bytes, void *stream,
                              unsigned int *completed, unsigned int *total);

int pccl_hip_graph_destroy(void *graph);

/* ---- errors ---------------------------------------------------------------- */
const char *pccl_hip_last_error(void);
const char *pccl_hip_version(void);

#ifdef __cplusplus
}
#endif
#endif
