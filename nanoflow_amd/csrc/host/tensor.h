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

  // Rows [first, first + count) as a view of the same layout; an empty range is the
  // reference's empty tensor (one "row" of zero columns) so that size() == 0.
  pllmTensor rowsView(size_t first, size_t count) const {
    if (count == 0) return pllmTensor(ptr + first * dim2, size_t(1), size_t(0), layout);
    return pllmTensor(ptr + first * dim2, count, dim2, layout);
  }

  pllmTensor subtensor(size_t startDim1, size_t dim1Count) const {
    if (startDim1 >= dim1 || dim1Count > dim1 - startDim1)
      throw std::out_of_range("subtensor: rows " + std::to_string(startDim1) + "+" + std::to_string(dim1Count) +
                              " of a tensor " + shapeString());
    return pllmTensor(ptr + startDim1 * dim2, dim1Count, dim2, layout);
  }
  pllmTensor subtensor(size_t startDim1) const {
    return pllmTensor(ptr + startDim1 * dim2, dim1 - startDim1, dim2, layout);
  }

  bool checkShape(const pllmTensor<T>& other) const {
    return layout == other.layout && dim1 == other.dim1 && dim2 == other.dim2;
  }
  bool assertShape(const pllmTensor<T>& other) const {
    if (checkShape(other)) return true;
    NF_LOG_ERROR("Shape mismatch: %s vs %s", shapeString().c_str(), other.shapeString().c_str());
    return false;
  }
  std::string shapeString() const {
    std::ostringstream os;
    os << '[' << dim1 << 'x' << dim2 << ' ' << toString(layout) << ']';
    return os.str();
  }
  // a row-major tensor is split along ROW, a column-major one along COLUMN: the enumerators pair up
  bool sameDirection(PllmDimension dim) const {
    return (dim == PllmDimension::ROW) == (layout == PllmLayout::ROW_MAJOR);
  }

  // The share of rank `rank` when dim1 is dealt out in nranks equal runs; what does not divide
  // goes to the last rank.
  pllmTensor<T> getSubTensor(int rank, int nranks, PllmDimension dim) const {
    assert(sameDirection(dim));
    const size_t each = dim1 / nranks, first = each * rank;
    return pllmTensor<T>{ptr + first * dim2, rank + 1 == nranks ? dim1 - first : each, dim2, layout};
  }

  // Consecutive pieces of the given lengths along dim1, which they must add up to.
  template <std::integral... Lens>
  std::array<pllmTensor<T>, sizeof...(Lens)> splitTensor(PllmDimension dim, Lens... lens) const {
    assert(sameDirection(dim));
    constexpr size_t N = sizeof...(Lens);
    const size_t want[N] = {static_cast<size_t>(lens)...};
    std::array<pllmTensor<T>, N> pieces;
    size_t first = 0;
    for (size_t i = 0; i < N; first += want[i++]) pieces[i] = rowsView(first, want[i]);
    assert(first == dim1 && "the lengths of the pieces must add up to the tensor's length");
    return pieces;
  }

  // Overlapping pieces: piece i starts where the lengths before it end and is lens[i] + suffix
  // long (n requests own n + 1 entries of an indptr array, the last shared with the next piece).
  template <size_t N, std::unsigned_integral TLen>
  std::array<pllmTensor<T>, N> splitTensor(PllmDimension dim, const std::span<TLen, N>& lens,
                                           TLen suffix = 0) const {
    assert(sameDirection(dim));
    std::array<pllmTensor<T>, N> pieces;
    size_t first = 0;
    for (size_t i = 0; i < N; first += lens[i++]) pieces[i] = rowsView(first, size_t(lens[i]) + suffix);
    assert((first + suffix) * dim2 == size() && "lengths plus the suffix must cover the tensor");
    return pieces;
  }

  // The same with a suffix of its own for every piece.
  template <size_t N, std::unsigned_integral TLen>
  std::array<pllmTensor<T>, N> splitTensor(PllmDimension dim, const std::span<TLen, N>& lens,
                                           const std::span<TLen, N>& suffix) const {
    assert(sameDirection(dim));
    std::array<pllmTensor<T>, N> pieces;
    size_t first = 0;
    for (size_t i = 0; i < N; first += lens[i++]) pieces[i] = rowsView(first, size_t(lens[i]) + suffix[i]);
    assert((first + suffix[N - 1]) * dim2 == size() && "lengths plus the last suffix must cover the tensor");
    return pieces;
  }

  pllmTensor<T> slice(PllmDimension dim, size_t start, size_t end) const {
    assert(sameDirection(dim));
    assert(start < end && end <= dim1);
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
  // the three layouts are the tag's last three '_'-separated fields
  std::array<std::string, 3> last;
  size_t end = input.size();
  for (int f = 2; f >= 0; --f) {
    const size_t us = end == 0 ? std::string::npos : input.rfind('_', end - 1);
    if (us == std::string::npos && f > 0)
      throw std::invalid_argument("GEMM tag \"" + input + "\" does not end in three layout fields");
    const size_t from = us == std::string::npos ? 0 : us + 1;
    last[f] = input.substr(from, end - from);
    end = us == std::string::npos ? 0 : us;
  }
  if (idx < 0 || idx > 2) throw std::out_of_range("GEMM tag layout index " + std::to_string(idx) + " (0..2)");
  if (last[idx] == "RowMajor") return PllmLayout::ROW_MAJOR;
  if (last[idx] == "ColumnMajor") return PllmLayout::COL_MAJOR;
  throw std::invalid_argument("GEMM tag \"" + input + "\": \"" + last[idx] + "\" is not a layout");
}
