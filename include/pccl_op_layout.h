/*
 * pccl_op_layout.h -- plain-data layouts shared by host code and device code.
 *
 * Field names, order, widths and offsets are those of the reference's
 *   include/base/chunk.h:10-14      ChunkMeta
 *   include/base/operator.h:7-17    RingBuffer
 *   include/base/operator.h:19-29   OperationLayoutHeader
 *   include/base/operator.h:31-38   GraphBufferLayout
 * (LP64).  They are restated as C structs so that the C ABI, the C++ host layer
 * (which re-exports them inside namespace engine_c) and the gfx950 kernels all
 * read the same bytes.  The reference only declares these structs and never
 * reads or writes them; the protocol notes beside the fields are this build's.
 */
#ifndef PCCL_OP_LAYOUT_H
#define PCCL_OP_LAYOUT_H

#ifdef __cplusplus
#include <cstddef>
#else
#include <stddef.h>
#endif

typedef unsigned char pccl_general_type; /* GeneralType, include/base/registry.h:12 */

/* Operand descriptor, 24 bytes. */
typedef struct pccl_chunk_meta {
  pccl_general_type dtype_; /* @0  */
  void *addr_;              /* @8  */
  long num_elems_;          /* @16 */
} pccl_chunk_meta;

/* Ready queue, 40 bytes.  Entries are pccl_queue_entry (elem_size_ == 8).
 * tail_ counts entries published, head_ counts entries claimed; both only grow
 * during a run and the run's last workgroup rewinds them.  producer_buffer_ and
 * consumer_buffer_ name the same device array when producer and consumer are
 * the same executor, which is the only case on one GPU.  producer_ and consumer_
 * carry the registry id given to pccl_hip_set_executor_id (the host layer passes
 * the id of "hip"; 0 if the C ABI is used without it). */
typedef struct pccl_ring_buffer {
  pccl_general_type producer_; /* @0  ExecutorType */
  pccl_general_type consumer_; /* @1  ExecutorType */
  int elem_size_;              /* @4  */
  int max_num_elems_;          /* @8  */
  int max_flush_time_;         /* @12 */
  int tail_;                   /* @16 */
  int head_;                   /* @20 */
  void *producer_buffer_;      /* @24 */
  void *consumer_buffer_;      /* @32 */
} pccl_ring_buffer;

/* One DAG node, 32 bytes.
 *   required_executors_  workgroup-sized parts the op is split into;
 *   remaining_executors_ parts not yet finished (counts down, then restored);
 *   pre_dependencies_    number of predecessors; constant during a run.  Device
 *                        code counts the predecessors that have finished on a
 *                        word of its own per op (outside this struct, alone on a
 *                        cache line) and runs the op when that count equals
 *                        this field;
 *   executor_type_       registry id of the executor that runs the op (see
 *                        pccl_ring_buffer::producer_);
 *   op_buffer_/op_size_  payload: pccl_op_payload, at most 255 bytes;
 *   next_op_uids_head_   num_next_ops_ successor uids. */
typedef struct pccl_operation_layout_header {
  int op_uid_;                      /* @0  */
  int required_executors_;          /* @4  */
  int remaining_executors_;         /* @8  */
  unsigned char pre_dependencies_;  /* @12 */
  pccl_general_type executor_type_; /* @13 */
  unsigned char op_size_;           /* @14 */
  unsigned char num_next_ops_;      /* @15 */
  void *op_buffer_;                 /* @16 */
  int *next_op_uids_head_;          /* @24 */
} pccl_operation_layout_header;

/* Whole program, 48 bytes. */
typedef struct pccl_graph_buffer_layout {
  unsigned int *completed_operator;         /* @0  */
  unsigned int *total_operator;             /* @8  */
  pccl_operation_layout_header **operators; /* @16 */
  unsigned int num_operators;               /* @24 */
  pccl_ring_buffer **ready_queues;          /* @32 */
  unsigned int num_queues;                  /* @40 */
} pccl_graph_buffer_layout;

/* Payload behind op_buffer_: 8-byte head + (n_in + n_out) operand descriptors,
 * inputs first.  8 + 10*24 = 248 <= 255 keeps op_size_ in its unsigned char,
 * so an op carries at most 10 operands in all (e.g. 8 inputs + 2 outputs). */
typedef struct pccl_op_payload {
  unsigned char primitive_; /* enum pccl_primitive */
  unsigned char compute_;   /* enum pccl_compute   */
  unsigned char n_in_;
  unsigned char n_out_;
  unsigned char pre_dependencies_; /* copy of the header's field */
  unsigned char part_preds_;       /* of those, dependencies that are met part by part (see below) */
  unsigned char part_nexts_;       /* successors that this op releases part by part; they come
                                      first in next_op_uids_head_ */
  unsigned char num_next_ops_;     /* copy of the header's field */
  pccl_chunk_meta chunks_[10];
} pccl_op_payload;

#define PCCL_MAX_OP_CHUNKS 10

/* Part-by-part dependencies.  When op B depends on op A, both are cut into the same number of
 * parts over the same number of bytes, and every operand of A that B's operands overlap
 * (with a write on either side) starts at the same address as the operand of B it overlaps,
 * then part p of B needs only part p of A, not all of A; the executor then lets B's part p
 * start as soon as A's part p is complete (and all of B's other dependencies are), which is
 * what lets a chain of large ops stream instead of draining between ops.  The same must hold
 * for every op still possibly in flight behind A through such edges; otherwise the
 * dependency stays whole-op.  (A and B sharing no bytes at all, a dependency that only orders
 * them, counts as "every overlap lines up".)  The observable result is that of whole-op
 * dependencies: memory ends as if the ops had run one after the other, B is complete only
 * after A is, and so is every NOTIFY behind B. */

/* Ready-queue entry: which op, which of its required_executors_ parts. */
typedef struct pccl_queue_entry {
  int op_uid;
  int part;
} pccl_queue_entry;

#ifdef __cplusplus
static_assert(sizeof(pccl_chunk_meta) == 24 && offsetof(pccl_chunk_meta, addr_) == 8 &&
              offsetof(pccl_chunk_meta, num_elems_) == 16, "ChunkMeta layout");
static_assert(sizeof(pccl_ring_buffer) == 40 && offsetof(pccl_ring_buffer, tail_) == 16 &&
              offsetof(pccl_ring_buffer, head_) == 20 &&
              offsetof(pccl_ring_buffer, producer_buffer_) == 24, "RingBuffer layout");
static_assert(sizeof(pccl_operation_layout_header) == 32 &&
              offsetof(pccl_operation_layout_header, pre_dependencies_) == 12 &&
              offsetof(pccl_operation_layout_header, num_next_ops_) == 15 &&
              offsetof(pccl_operation_layout_header, op_buffer_) == 16 &&
              offsetof(pccl_operation_layout_header, next_op_uids_head_) == 24,
              "OperationLayoutHeader layout");
static_assert(sizeof(pccl_graph_buffer_layout) == 48 &&
              offsetof(pccl_graph_buffer_layout, num_operators) == 24 &&
              offsetof(pccl_graph_buffer_layout, ready_queues) == 32 &&
              offsetof(pccl_graph_buffer_layout, num_queues) == 40, "GraphBufferLayout layout");
static_assert(sizeof(pccl_op_payload) == 248, "payload must fit op_size_ (unsigned char)");
static_assert(sizeof(pccl_queue_entry) == 8, "queue entry");
#endif

#endif
