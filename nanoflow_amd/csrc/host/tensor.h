// pllmTensor: a non-owning (pointer, rows, cols, layout) view with the slicing helpers the
// pipelines use to carve nano-batches and per-launch metadata out of shared buffers.
// Same names and semantics as the reference's pipeline/include/tensor.cuh:17-300.
#pragma once
#include <algorithm>
#include <array>
#include <cassert>
#include <concepts>
#include <cstdint>
#include <numeric>
#include <span>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

#include "helper.h"

using half = uint16_t;  // fp16 bit pattern; the host never does arithmetic on it

enum class PllmLayout { ROW_MAJOR, COL_MAJOR };
enum class PllmDimension { ROW, COLUMN };

inline std::string toString(PllmLayout layout) {
  return layout == PllmLayout::ROW_MAJOR ? "ROW_MAJOR" : "COL_MAJOR";
}
inline std::string toString(PllmDimension dim) {
  return dim == PllmDimension::ROW ? "ROW" : "COLUMN";
}

template <typename T>
struct pllmTensor {
  T* ptr = nullptr;
  size_t dim1 = 0;
  size_t dim2 = 0;
  PllmLayout layout = PllmLayout::ROW_MAJOR;

  pllmTensor() = default;
  pllmTensor(T* ptr, size_t dim1, size_t dim2, PllmLayout layout)
      : ptr(ptr), dim1(dim1), dim2(dim2), layout(layout) {}
  pllmTensor(T* ptr, int dim1, int dim2, PllmLayout layout)
      : ptr(ptr), dim1(dim1), dim2(dim2), layout(layout) {
    assert(dim1 >= 0 && dim2 >= 0);
  }
  pllmTensor(T* ptr, size_t length) : ptr(ptr), dim1(length), dim2(1) {}
  pllmTensor(T* ptr, int length) : ptr(ptr), dim1(length), dim2(1) { assert(length >= 0); }

  size_t dimC() const { return dim2; }
  size_t size() const { return dim1 * dim2; }
  size_t bytes() const { return size() * sizeof(T); }

  pllmTensor subtensor(size_t startDim1, size_t dim1Count) const {
    if (startDim1 >= dim1) throw std::out_of_range("Invalid start position for subtensor.");
    if (startDim1 + dim1Count > dim1) throw std::out_of_range("Invalid row count for subtensor.");
    return pllmTensor(ptr + startDim1 * dim2, dim1Count, dim2, layout);
  }
  pllmTensor subtensor(size_t startDim1) const {
    return pllmTensor(ptr + startDim1 * dim2, dim1 - startDim1, dim2, layout);
  }

  bool checkShape(const pllmTensor<T>& other) const {
    return dim1 == other.dim1 && dim2 == other.dim2 && layout == other.layout;
  }
  bool assertShape(const pllmTensor<T>& other) const {
    bool ret = checkShape(other);
    if (!ret)
      NF_LOG_ERROR("Shape mismatch: %s vs %s", shapeString().c_str(), other.shapeString().c_str());
    return ret;
  }
  std::string shapeString() const {
    return "[" + std::to_string(dim1) + "x" + std::to_string(dim2) + " " + toString(layout) + "]";
  }
  bool sameDirection(PllmDimension dim) const {
    return static_cast<int>(dim) == static_cast<int>(layout);
  }

  // rank-th of nranks equal row chunks (the last takes the remainder)
  pllmTensor<T> getSubTensor(int rank, int nranks, PllmDimension dim) const {
    assert(sameDirection(dim));
    size_t chunk = dim1 / nranks;
    size_t final_chunk = chunk + (rank == nranks - 1 ? dim1 % nranks : 0);
    return pllmTensor<T>{ptr + rank * chunk * dim2, final_chunk, dim2, layout};
  }

  // Split along rows into consecutive pieces of the given lengths.  A zero length yields
  // the empty tensor {ptr, 1, 0}.
  template <std::integral... Lens>
  std::array<pllmTensor<T>, sizeof...(Lens)> splitTensor(PllmDimension dim, Lens... lens) const {
    assert(sameDirection(dim));
    [[maybe_unused]] size_t total = (size_t(0) + ... + size_t(lens));
    assert(dim1 == total && "Subtensor length sum mismatches with the input tensor");
    size_t i = 0, offset = 0;
    std::array<pllmTensor<T>, sizeof...(Lens)> ret;
    ((ret[i++] = (static_cast<size_t>(lens) == 0
                      ? pllmTensor<T>{ptr + offset, size_t(1), size_t(0), layout}
                      : pllmTensor<T>{ptr + offset, static_cast<size_t>(lens), dim2, layout}),
      offset += lens * dim2),
     ...);
    return ret;
  }

  // Split with an overlapping suffix: piece i is lens[i] + suffix rows long and piece i+1
  // starts lens[i] rows later (used for indptr arrays: n requests need n+1 entries).
  template <size_t N, std::unsigned_integral TLen>
  std::array<pllmTensor<T>, N> splitTensor(PllmDimension dim, const std::span<TLen, N>& lens,
                                           TLen suffix = 0) const {
    assert(sameDirection(dim));
    assert(size() == std::accumulate(lens.begin(), lens.end(), size_t(0)) + suffix &&
           "Subspan length sum mismatches with the input span");
    size_t offset = 0;
    std::array<pllmTensor<T>, N> ret;
    for (size_t i = 0; i < N; ++i) {
      size_t l = lens[i];
      ret[i] = (l + suffix == 0) ? pllmTensor<T>{ptr + offset, size_t(1), size_t(0), layout}
                                 : pllmTensor<T>{ptr + offset, l + suffix, dim2, layout};
      offset += l * dim2;
    }
    return ret;
  }

  // Per-piece suffix lengths.
  template <size_t N, std::unsigned_integral TLen>
  std::array<pllmTensor<T>, N> splitTensor(PllmDimension dim, const std::span<TLen, N>& lens,
                                           const std::span<TLen, N>& suffix) const {
    assert(sameDirection(dim));
    assert(size() == std::accumulate(lens.begin(), lens.end(), size_t(0)) + suffix[N - 1] &&
           "Subspan length sum mismatches with the input span");
    size_t offset = 0;
    std::array<pllmTensor<T>, N> ret;
    for (size_t i = 0; i < N; ++i) {
      size_t l = lens[i];
      ret[i] = (l + suffix[i] == 0) ? pllmTensor<T>{ptr + offset, size_t(1), size_t(0), layout}
                                    : pllmTensor<T>{ptr + offset, l + suffix[i], dim2, layout};
      offset += l * dim2;
    }
    return ret;
  }

  pllmTensor<T> slice(PllmDimension dim, size_t start, size_t end) const {
    assert(sameDirection(dim));
    assert(end <= dim1 && start < end);
    return pllmTensor<T>{ptr + start * dim2, end - start, dim2, layout};
  }
};

template <typename Tsrc, typename Tdst>
inline pllmTensor<Tdst> tensor_cast(pllmTensor<Tsrc> src) {
  static_assert(sizeof(Tdst) == sizeof(Tsrc));
  return pllmTensor<Tdst>{reinterpret_cast<Tdst*>(src.ptr), src.dim1, src.dim2, src.layout};
}

// Fields of a GEMM tag "ctaM_ctaN_ctaK_warpM_warpN_warpK_splitK_stages_{Row|Column}Major x3"
// (pipeline/include/gemmShape.cuh:5-6).  idx 0/1/2 = layout of A / B / output.
inline PllmLayout getMajorType(const std::string& input, int idx) {
  std::stringstream ss(input);
  std::string token;
  std::vector<std::string> parts;
  while (std::getline(ss, token, '_')) parts.push_back(token);
  auto it = std::find_if(parts.begin(), parts.end(), [](const std::string& s) {
    return s == "RowMajor" || s == "ColumnMajor";
  });
  if (it == parts.end()) throw std::invalid_argument("No major types found");
  size_t start = std::distance(parts.begin(), it);
  if (idx < 0 || start + idx >= parts.size()) throw std::out_of_range("Index is out of range");
  const std::string& major = parts[start + idx];
  if (major == "RowMajor") return PllmLayout::ROW_MAJOR;
  if (major == "ColumnMajor") return PllmLayout::COL_MAJOR;
  throw std::invalid_argument("Invalid major type");
}
