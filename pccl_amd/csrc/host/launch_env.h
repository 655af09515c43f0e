// launch_env.h -- snapshot of the process environment plus the list of option
// names plugins advertise, and a small stderr logger.
//
// LaunchEnvironments follows the reference's include/common/environ.h:11-37 /
// csrc/common/environ.cc:8-29: the environment is captured once at first use,
// getEnv() returns "" for an unset name, plugins call registerOpt() from their
// static initialisers and listOpt() reports the names.
// The logger honours the reference's PCCL_LOG_LEVEL (TRACE..CRITICAL, default
// WARN; csrc/common/logging.cc:8-28) and writes to stderr only.
#pragma once

#include <string>
#include <vector>

namespace engine_c::utils {

class LaunchEnvironments {
public:
  static std::string getEnv(const std::string &name);
  static void registerOpt(const std::string &name);
  static std::vector<std::string> listOpt();
};

enum class LogLevel { Trace = 0, Debug, Info, Warn, Error, Critical, Off };
LogLevel logLevel();
void logMessage(LogLevel level, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

}  // namespace engine_c::utils

#define PCCL_LOG_INFO(...) ::engine_c::utils::logMessage(::engine_c::utils::LogLevel::Info, __VA_ARGS__)
#define PCCL_LOG_WARN(...) ::engine_c::utils::logMessage(::engine_c::utils::LogLevel::Warn, __VA_ARGS__)
#define PCCL_LOG_ERROR(...) ::engine_c::utils::logMessage(::engine_c::utils::LogLevel::Error, __VA_ARGS__)
