#include "core/common.h"

#include <cstdio>
#include <cstdlib>

namespace dragon {

namespace {
void AbortingFatalHandler(const string&) { std::abort(); }
FatalHandler g_fatal_handler = AbortingFatalHandler;
int g_log_severity = INFO;
const char* kSeverityNames[] = {"DEBUG", "INFO", "WARNING", "ERROR", "FATAL"};
} // namespace

FatalHandler SetFatalHandler(FatalHandler handler) {
  FatalHandler previous = g_fatal_handler;
  g_fatal_handler = handler ? handler : AbortingFatalHandler;
  return previous;
}

void ThrowingFatalHandler(const string& message) { throw FatalError(message); }

void SetLogSeverity(int severity) { g_log_severity = severity; }

MessageLogger::MessageLogger(const char* file, int line, int severity) : severity_(severity) {
  const char* base = std::strrchr(file, '/');
  stream_ << kSeverityNames[severity] << " " << (base ? base + 1 : file) << ":" << line << "] ";
}

MessageLogger::~MessageLogger() noexcept(false) {
  if (severity_ < g_log_severity) return;
  const string message = stream_.str();
  std::fprintf(stderr, "%s\n", message.c_str());
  std::fflush(stderr);
  if (severity_ == FATAL) g_fatal_handler(message);
}

} // namespace dragon
