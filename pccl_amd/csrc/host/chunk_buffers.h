// chunk_buffers.h -- operand descriptors and the per-device workspace registry.
//
// ChunkMeta / BufferMeta keep the fields of the reference's
// include/base/chunk.h:10-20; ChunkMeta is the very struct the device kernels
// read (pccl_chunk_meta).  BufferManager keeps regBuffer / getDevBuffer
// (chunk.h:42-46; declared in the reference, never defined).  The cross-rank
// half of the reference's class (GlobalBufferIdentifier, DataWorkspaceMeta,
// regCommResource, assignBuffer: chunk.h:22-36,48-53) exchanges handles between
// processes and is not part of this single-GPU build.
#pragma once

#include <map>
#include <mutex>
#include <tuple>

#include "pccl_op_layout.h"
#include "type_registry.h"

namespace engine_c {

using ChunkMeta = ::pccl_chunk_meta;  // {DataType dtype_; void *addr_; long num_elems_;}

struct BufferMeta {
  DeviceType device_;
  int buffer_idx_;
  long size_;
};

class BufferManager {
public:
  BufferManager() = default;

  // Records the workspace of one device type: `buf` of `size` bytes and the
  // `slots` int signal slots at `signals` (engine.cc:69-71,77-79 pass
  // buf + WORKSPACE_SIZE).  A second registration for the same type replaces
  // the first.
  void regBuffer(void *buf, long size, int *signals, long slots, int rank, GeneralType type);

  // (workspace, signals) of a device type; throws std::runtime_error if none.
  std::tuple<void *, void *> getDevBuffer(GeneralType type);

  bool hasDevBuffer(GeneralType type);
  long getDevBufferSize(GeneralType type);
  BufferMeta getMeta(GeneralType type);

private:
  struct Entry {
    void *buf;
    long size;
    int *signals;
    long slots;
    int rank;
    int index;
  };
  std::mutex mu_;
  std::map<GeneralType, Entry> entries_;
};

}  // namespace engine_c
