// Error handling and logging for the host library.
// Behaviour follows the reference's helper.h (pipeline/include/helper.h:39-61): a GPU runtime
// failure prints the call site and terminates the process.
#pragma once
#include <hip/hip_runtime_api.h>

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <string>

namespace nflog {
enum Level { TRACE = 0, INFO = 1, WARN = 2, ERROR = 3, OFF = 4 };
// Level comes from NANOFLOW_LOG (trace|info|warn|error|off); default warn.
int level();
void write(Level lvl, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
}  // namespace nflog

#define NF_LOG_INFO(...)  do { if (nflog::level() <= nflog::INFO) nflog::write(nflog::INFO, __VA_ARGS__); } while (0)
#define NF_LOG_WARN(...)  do { if (nflog::level() <= nflog::WARN) nflog::write(nflog::WARN, __VA_ARGS__); } while (0)
#define NF_LOG_ERROR(...) do { if (nflog::level() <= nflog::ERROR) nflog::write(nflog::ERROR, __VA_ARGS__); } while (0)

#define HIP_CHECK(call)                                                                   \
  do {                                                                                    \
    hipError_t err_ = (call);                                                             \
    if (err_ != hipSuccess) {                                                             \
      std::fprintf(stderr, "HIP error at %s:%d code=%d(%s) \"%s\"\n", __FILE__, __LINE__, \
                   (int)err_, hipGetErrorString(err_), #call);                            \
      std::exit(EXIT_FAILURE);                                                            \
    }                                                                                     \
  } while (0)

// Kernel-layer status -> same policy as a failing GEMM library call in the reference
// (CUTLASS_CHECK, pipeline/include/helper.h:50-61): report and terminate.
#define NF_KERNEL_CHECK(call)                                                              \
  do {                                                                                     \
    int rc_ = (call);                                                                      \
    if (rc_ != 0) {                                                                        \
      std::fprintf(stderr, "kernel layer error at %s:%d rc=%d: %s\n", __FILE__, __LINE__,  \
                   rc_, nf_last_error());                                                  \
      std::exit(EXIT_FAILURE);                                                             \
    }                                                                                      \
  } while (0)
