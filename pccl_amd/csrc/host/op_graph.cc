#include "op_graph.h"

#include <stdexcept>

#include "executor.h"

namespace engine_c {

RegisteredOp::~RegisteredOp() {
  if (graph && executor) executor->destroyGraph(graph);
}

std::shared_ptr<RegisteredOp> OperatorManager::add(const std::string &name, Schedule schedule) {
  auto op = std::make_shared<RegisteredOp>();
  op->schedule = std::move(schedule);
  std::lock_guard<std::mutex> lock(mu_);
  ops_[name] = op;
  return op;
}

std::shared_ptr<RegisteredOp> OperatorManager::get(const std::string &name) {
  std::lock_guard<std::mutex> lock(mu_);
  auto it = ops_.find(name);
  if (it == ops_.end()) throw std::runtime_error("no operator registered under the name '" + name + "'");
  return it->second;
}

bool OperatorManager::has(const std::string &name) {
  std::lock_guard<std::mutex> lock(mu_);
  return ops_.count(name) != 0;
}

void OperatorManager::remove(const std::string &name) {
  std::lock_guard<std::mutex> lock(mu_);
  ops_.erase(name);
}

}  // namespace engine_c
