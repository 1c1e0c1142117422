// Tensor dumps for debugging a schedule: the first rows x cols elements of an operator's
// operands, printed after the operator has run.  Output format of the reference's
// pipeline/include/tensorLogger.cuh:15-60 ("--------Tensor name (row a->b, col c->d)------------"
// followed by one comma-separated line per row).  The reference compiles the dumps in or out
// (ENABLE_LOGGING, operatorWrapper.cuh:146-156); here they are switched at run time by the
// environment variable NANOFLOW_TENSOR_LOG (a file path, or "stderr"), read when a pipeline
// is created, and cost one predictable branch per operator when off.
#pragma once
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <type_traits>
#include <vector>

#include "helper.h"
#include "tensor.h"

namespace tensorlog {

struct Sink {
  FILE* file = nullptr;
  bool owned = false;
};
inline Sink& sink() {
  static Sink s;
  return s;
}
inline bool enabled() { return sink().file != nullptr; }

// (Re)reads NANOFLOW_TENSOR_LOG; an unset or empty variable switches the dumps off.
inline void configure() {
  Sink& s = sink();
  if (s.file && s.owned) std::fclose(s.file);
  s = Sink{};
  const char* path = std::getenv("NANOFLOW_TENSOR_LOG");
  if (!path || !*path) return;
  if (std::string(path) == "stderr") {
    s.file = stderr;
    return;
  }
  s.file = std::fopen(path, "a");
  s.owned = s.file != nullptr;
  if (!s.file) NF_LOG_ERROR("NANOFLOW_TENSOR_LOG: cannot open %s", path);
}

// A stream under graph capture cannot be waited for: such launches are not dumped.
inline bool capturing(hipStream_t stream) {
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &st) != hipSuccess) return true;
  return st != hipStreamCaptureStatusNone;
}

// fp16 bit pattern (the host's `half`) to float
inline float half_to_float(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu, man = h & 0x3ffu, bits;
  if (exp == 0x1fu) {
    bits = sign | 0x7f800000u | (man << 13);
  } else if (exp) {
    bits = sign | ((exp + 112u) << 23) | (man << 13);
  } else if (man) {
    int e = -1;
    do { man <<= 1; ++e; } while (!(man & 0x400u));
    bits = sign | ((uint32_t)(112 - e) << 23) | ((man & 0x3ffu) << 13);
  } else {
    bits = sign;
  }
  float f;
  std::memcpy(&f, &bits, 4);
  return f;
}
inline void print_element(FILE* f, half v) { std::fprintf(f, "%g", (double)half_to_float(v)); }
inline void print_element(FILE* f, float v) { std::fprintf(f, "%g", (double)v); }
inline void print_element(FILE* f, int32_t v) { std::fprintf(f, "%d", v); }

// Waits for `stream`, then prints rows [start_row, start_row + rows) x cols [start_col, start_col + cols)
// of `t` (clipped to its shape).  The storage is read as dim1 rows of dim2 elements whatever the
// layout label says, as the reference does; a vector (dim2 == 1) is printed as one row.
template <typename T>
void log_tensor(hipStream_t stream, const std::string& owner, const char* tensor_name, pllmTensor<T> t,
                size_t rows = 1, size_t cols = 20, size_t start_row = 0, size_t start_col = 0) {
  FILE* f = sink().file;
  if (!f) return;
  if (t.dim2 == 1 && t.dim1 > 1) t = pllmTensor<T>(t.ptr, size_t(1), t.dim1, t.layout);  // a vector: one row
  if (!t.ptr || t.size() == 0 || start_row >= t.dim1 || start_col >= t.dim2) {
    std::fprintf(f, "--------Tensor %s%s (empty)------------\n", owner.c_str(), tensor_name);
    return;
  }
  if (rows > t.dim1 - start_row) rows = t.dim1 - start_row;
  if (cols > t.dim2 - start_col) cols = t.dim2 - start_col;
  std::vector<T> host(rows * cols);
  HIP_CHECK(hipStreamSynchronize(stream));
  HIP_CHECK(hipMemcpy2D(host.data(), cols * sizeof(T), t.ptr + start_row * t.dim2 + start_col, t.dim2 * sizeof(T),
                        cols * sizeof(T), rows, hipMemcpyDeviceToHost));
  std::fprintf(f, "--------Tensor %s%s (row %zu->%zu, col %zu->%zu)------------\n", owner.c_str(), tensor_name,
               start_row, start_row + rows, start_col, start_col + cols);
  for (size_t r = 0; r < rows; ++r) {
    for (size_t c = 0; c < cols; ++c) {
      if (c) std::fputs(", ", f);
      print_element(f, host[r * cols + c]);
    }
    std::fputc('\n', f);
  }
  std::fflush(f);
}

}  // namespace tensorlog
