#include "type_registry.h"

#include <map>
#include <memory>
#include <mutex>
#include <stdexcept>
#include <unordered_map>
#include <vector>

namespace engine_c {

struct TypeRegistry::State {
  std::mutex mu;
  std::unordered_map<std::string, GeneralType> id_of;
  // ids are dense, so names and kinds are indexable; deque-like stability is not
  // needed because string_views handed out point into heap strings
  std::vector<std::unique_ptr<std::string>> name_of;
  std::vector<Kind> kind_of;
  std::set<DeviceType> devices;
  std::map<ExecutorType, std::set<GeneralType>> compatible_types;
  std::map<GeneralType, std::set<ExecutorType>> compatible_executors;
};

// Function-local static: plugins register from their own static initialisers,
// which may run before any namespace-scope object of this file is constructed.
TypeRegistry::State &TypeRegistry::state() {
  static State *s = new State();  // never destroyed: plugins may outlive static teardown
  return *s;
}

GeneralType TypeRegistry::add(std::string_view name, Kind kind) {
  State &s = state();
  std::lock_guard<std::mutex> lock(s.mu);
  auto it = s.id_of.find(std::string(name));
  if (it != s.id_of.end()) {
    if (s.kind_of[it->second] != kind)
      throw std::runtime_error("TypeRegistry: '" + std::string(name) + "' is already registered as another kind");
    return it->second;
  }
  if (s.name_of.size() >= 256) throw std::runtime_error("TypeRegistry: all 256 ids are in use");
  const GeneralType id = static_cast<GeneralType>(s.name_of.size());
  s.name_of.push_back(std::make_unique<std::string>(name));
  s.kind_of.push_back(kind);
  s.id_of.emplace(std::string(name), id);
  if (kind == Kind::Device) s.devices.insert(id);
  return id;
}

PrimitiveType TypeRegistry::registerPrimitive(std::string_view n) { return add(n, Kind::Primitive); }
DataType TypeRegistry::registerDataType(std::string_view n) { return add(n, Kind::Data); }
ComputeType TypeRegistry::registerComputeType(std::string_view n) { return add(n, Kind::Compute); }
DeviceType TypeRegistry::registerDeviceType(std::string_view n) { return add(n, Kind::Device); }
ExecutorType TypeRegistry::registerExecutorType(std::string_view n) { return add(n, Kind::Executor); }

void TypeRegistry::registerCompatibility(std::string_view executor_name, std::string_view type_name) {
  State &s = state();
  std::lock_guard<std::mutex> lock(s.mu);
  auto e = s.id_of.find(std::string(executor_name));
  auto t = s.id_of.find(std::string(type_name));
  if (e == s.id_of.end() || s.kind_of[e->second] != Kind::Executor)
    throw std::runtime_error("TypeRegistry: unknown executor '" + std::string(executor_name) + "'");
  if (t == s.id_of.end()) throw std::runtime_error("TypeRegistry: unknown type '" + std::string(type_name) + "'");
  s.compatible_types[e->second].insert(t->second);
  s.compatible_executors[t->second].insert(e->second);
}

std::string_view TypeRegistry::getTypeName(GeneralType type) {
  State &s = state();
  std::lock_guard<std::mutex> lock(s.mu);
  if (type >= s.name_of.size()) throw std::out_of_range("TypeRegistry: unknown type id " + std::to_string(type));
  return *s.name_of[type];
}

GeneralType TypeRegistry::getTypeId(std::string_view name) {
  State &s = state();
  std::lock_guard<std::mutex> lock(s.mu);
  auto it = s.id_of.find(std::string(name));
  if (it == s.id_of.end()) throw std::out_of_range("TypeRegistry: unknown type name '" + std::string(name) + "'");
  return it->second;
}

bool TypeRegistry::hasType(std::string_view name) {
  State &s = state();
  std::lock_guard<std::mutex> lock(s.mu);
  return s.id_of.count(std::string(name)) != 0;
}

TypeRegistry::Kind TypeRegistry::getKind(GeneralType type) {
  State &s = state();
  std::lock_guard<std::mutex> lock(s.mu);
  if (type >= s.kind_of.size()) throw std::out_of_range("TypeRegistry: unknown type id " + std::to_string(type));
  return s.kind_of[type];
}

const std::set<DeviceType> &TypeRegistry::getDeviceTypes() { return state().devices; }

const std::set<GeneralType> &TypeRegistry::getCompatibleTypes(ExecutorType executor_type) {
  static const std::set<GeneralType> none;
  State &s = state();
  std::lock_guard<std::mutex> lock(s.mu);
  auto it = s.compatible_types.find(executor_type);
  return it == s.compatible_types.end() ? none : it->second;
}

const std::set<ExecutorType> &TypeRegistry::getCompatibleExecutors(GeneralType type) {
  static const std::set<ExecutorType> none;
  State &s = state();
  std::lock_guard<std::mutex> lock(s.mu);
  auto it = s.compatible_executors.find(type);
  return it == s.compatible_executors.end() ? none : it->second;
}

void TypeRegistry::clear() {
  State &s = state();
  std::lock_guard<std::mutex> lock(s.mu);
  s.id_of.clear();
  s.name_of.clear();
  s.kind_of.clear();
  s.devices.clear();
  s.compatible_types.clear();
  s.compatible_executors.clear();
}

}  // namespace engine_c
