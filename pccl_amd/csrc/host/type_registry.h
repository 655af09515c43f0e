// type_registry.h -- string <-> small-integer ids for primitives, data types,
// compute types, device types and executor types, plus an executor/type
// compatibility relation.
//
// Interface of the reference's include/base/registry.h:12-43 (declared there,
// never defined: csrc/base/registry.cc:1-5 is an empty namespace).  As in the
// reference all kinds share ONE id counter (registry.h:79), so at most 256 names
// exist in total and an id identifies its kind.  Registering a name twice
// returns the id it already has.
#pragma once

#include <set>
#include <string>
#include <string_view>

namespace engine_c {

using GeneralType = unsigned char;
using PrimitiveType = GeneralType;
using DataType = GeneralType;
using ComputeType = GeneralType;
using DeviceType = GeneralType;
using ExecutorType = GeneralType;

struct TypeCompatibility {
  ExecutorType executor_type;
  GeneralType target_type;
  bool is_compatible;
};

class TypeRegistry {
public:
  enum class Kind : unsigned char { Primitive, Data, Compute, Device, Executor };

  static PrimitiveType registerPrimitive(std::string_view name);
  static DataType registerDataType(std::string_view name);
  static ComputeType registerComputeType(std::string_view name);
  static DeviceType registerDeviceType(std::string_view name);
  static ExecutorType registerExecutorType(std::string_view name);
  // Both names must be registered already; throws std::runtime_error otherwise.
  static void registerCompatibility(std::string_view executor_name, std::string_view type_name);

  // Throws std::out_of_range for an unknown id / name.
  static std::string_view getTypeName(GeneralType type);
  static GeneralType getTypeId(std::string_view name);
  static bool hasType(std::string_view name);
  static Kind getKind(GeneralType type);

  static const std::set<DeviceType> &getDeviceTypes();
  static const std::set<GeneralType> &getCompatibleTypes(ExecutorType executor_type);
  static const std::set<ExecutorType> &getCompatibleExecutors(GeneralType type);

  // Forgets everything (tests only: plugins registered at load time disappear too).
  static void clear();

private:
  TypeRegistry() = default;
  struct State;
  static State &state();
  static GeneralType add(std::string_view name, Kind kind);
};

}  // namespace engine_c
