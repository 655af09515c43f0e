#include "chunk_buffers.h"

#include <stdexcept>
#include <string>

namespace engine_c {

void BufferManager::regBuffer(void *buf, long size, int *signals, long slots, int rank, GeneralType type) {
  if (!buf || size <= 0) throw std::runtime_error("BufferManager::regBuffer(): empty buffer");
  std::lock_guard<std::mutex> lock(mu_);
  auto it = entries_.find(type);
  const int index = it == entries_.end() ? (int)entries_.size() : it->second.index;
  entries_[type] = Entry{buf, size, signals, slots, rank, index};
}

std::tuple<void *, void *> BufferManager::getDevBuffer(GeneralType type) {
  std::lock_guard<std::mutex> lock(mu_);
  auto it = entries_.find(type);
  if (it == entries_.end())
    throw std::runtime_error("BufferManager::getDevBuffer(): no workspace for device type " + std::to_string(type));
  return {it->second.buf, (void *)it->second.signals};
}

bool BufferManager::hasDevBuffer(GeneralType type) {
  std::lock_guard<std::mutex> lock(mu_);
  return entries_.count(type) != 0;
}

long BufferManager::getDevBufferSize(GeneralType type) {
  std::lock_guard<std::mutex> lock(mu_);
  auto it = entries_.find(type);
  return it == entries_.end() ? 0 : it->second.size;
}

BufferMeta BufferManager::getMeta(GeneralType type) {
  std::lock_guard<std::mutex> lock(mu_);
  auto it = entries_.find(type);
  if (it == entries_.end())
    throw std::runtime_error("BufferManager::getMeta(): no workspace for device type " + std::to_string(type));
  return BufferMeta{type, it->second.index, it->second.size};
}

}  // namespace engine_c
