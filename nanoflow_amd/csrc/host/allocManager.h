// Bump allocator over a caller-owned buffer (the pipeline's tmp_buffer).
// Same interface as the reference's pipeline/include/allocManager.cuh:26-61; running past the
// end is a hard error in every build type (the reference asserts).
#pragma once
#include <span>

#include "tensor.h"

template <typename T>
class AllocationManager {
public:
  // size is in elements of T, not bytes
  AllocationManager(T* base, size_t size) : base(base), allocated(0), size(size) {}

  T* alloc(size_t n) {
    if (allocated + n > size) {
      std::fprintf(stderr, "AllocationManager: %zu + %zu elements exceed the buffer of %zu\n",
                   allocated, n, size);
      std::exit(EXIT_FAILURE);
    }
    T* ret = base + allocated;
    allocated += n;
    return ret;
  }
  // bytes of scratch at a 256-byte boundary of the buffer (nullptr for 0 bytes)
  void* allocBytes(size_t bytes) {
    if (bytes == 0) return nullptr;
    const size_t unit = 256 / sizeof(T);
    alloc((unit - allocated % unit) % unit);
    return alloc((bytes + sizeof(T) - 1) / sizeof(T));
  }
  std::span<T> allocSpan(size_t n) { return std::span<T>{alloc(n), n}; }
  pllmTensor<T> allocTensor(int M, int N, PllmLayout layout) {
    if (layout == PllmLayout::ROW_MAJOR) return pllmTensor<T>{alloc((size_t)M * N), M, N, layout};
    return pllmTensor<T>{alloc((size_t)M * N), N, M, layout};
  }
  size_t getAllocation() const { return allocated; }

private:
  T* base;
  size_t allocated;
  size_t size;
};
