// Error convention of the engine this layer plugs into: no exceptions, no status codes; an
// unrecoverable condition prints and exits with a code (reference: mllm/Utils/Log.hpp:59-64,
// codes mllm/Utils/Common.hpp:23-30). The handler is replaceable so tests can observe it.
#pragma once

#include <cstdio>
#include <cstdlib>
#include <functional>
#include <string>

namespace mllm {

enum ExitCode : int {  // NOLINT
  kSuccess = 0,
  kCoreError = 1,
  kAssert = 2,
  kIOError = 3,
  kHipError = 4,
  kShapeError = 5,
};

inline std::function<void(int, const std::string&)>& errorHandler() {
  static std::function<void(int, const std::string&)> h = [](int code, const std::string& msg) {
    std::fprintf(stderr, "[mllm][ERROR] %s\n", msg.c_str());
    std::fflush(stderr);
    std::exit(code);
  };
  return h;
}

template <typename... Args>
inline std::string formatMsg(const char* fmt, Args... args) {
  char buf[1024];
  std::snprintf(buf, sizeof buf, fmt, args...);
  return std::string(buf);
}
inline std::string formatMsg(const char* fmt) { return std::string(fmt); }

}  // namespace mllm

#define MLLM_ERROR_EXIT(code, ...) ::mllm::errorHandler()((code), ::mllm::formatMsg(__VA_ARGS__))
#define MLLM_WARN(...) std::fprintf(stderr, "[mllm][WARN] %s\n", ::mllm::formatMsg(__VA_ARGS__).c_str())
#define MLLM_INFO(...) std::fprintf(stderr, "[mllm][INFO] %s\n", ::mllm::formatMsg(__VA_ARGS__).c_str())
#define MLLM_RT_ASSERT(expr)                                                                  \
  do {                                                                                        \
    if (!(expr)) MLLM_ERROR_EXIT(::mllm::kAssert, "assert failed: %s (%s:%d)", #expr, __FILE__, __LINE__); \
  } while (0)
#define MLLM_RT_ASSERT_EQ(a, b) MLLM_RT_ASSERT((a) == (b))
