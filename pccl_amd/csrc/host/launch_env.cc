#include "launch_env.h"

#include <algorithm>
#include <cstdarg>
#include <cstdio>
#include <map>
#include <mutex>

extern char **environ;

namespace engine_c::utils {

namespace {
struct EnvState {
  std::mutex mu;
  bool captured = false;
  std::map<std::string, std::string> vars;
  std::vector<std::string> opts;
};

EnvState &env() {
  static EnvState *s = new EnvState();
  return *s;
}

void capture_locked(EnvState &s) {
  if (s.captured) return;
  s.captured = true;
  for (char **e = environ; e && *e; ++e) {
    std::string kv(*e);
    const size_t eq = kv.find('=');
    if (eq != std::string::npos) s.vars[kv.substr(0, eq)] = kv.substr(eq + 1);
  }
}
}  // namespace

std::string LaunchEnvironments::getEnv(const std::string &name) {
  EnvState &s = env();
  std::lock_guard<std::mutex> lock(s.mu);
  capture_locked(s);
  auto it = s.vars.find(name);
  return it == s.vars.end() ? std::string() : it->second;
}

void LaunchEnvironments::registerOpt(const std::string &name) {
  EnvState &s = env();
  std::lock_guard<std::mutex> lock(s.mu);
  if (std::find(s.opts.begin(), s.opts.end(), name) == s.opts.end()) s.opts.push_back(name);
}

std::vector<std::string> LaunchEnvironments::listOpt() {
  EnvState &s = env();
  std::lock_guard<std::mutex> lock(s.mu);
  return s.opts;
}

LogLevel logLevel() {
  static const LogLevel level = [] {
    std::string v = LaunchEnvironments::getEnv("PCCL_LOG_LEVEL");
    std::transform(v.begin(), v.end(), v.begin(), [](unsigned char c) { return (char)toupper(c); });
    if (v == "TRACE") return LogLevel::Trace;
    if (v == "DEBUG") return LogLevel::Debug;
    if (v == "INFO") return LogLevel::Info;
    if (v == "ERROR") return LogLevel::Error;
    if (v == "CRITICAL") return LogLevel::Critical;
    if (v == "OFF") return LogLevel::Off;
    return LogLevel::Warn;
  }();
  return level;
}

void logMessage(LogLevel level, const char *fmt, ...) {
  if (level < logLevel()) return;
  static const char *names[] = {"trace", "debug", "info", "warn", "error", "critical", "off"};
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  fprintf(stderr, "[pccl][%s] %s\n", names[(int)level], buf);
}

}  // namespace engine_c::utils
