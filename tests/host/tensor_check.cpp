// Host-only check of pllmTensor's slicing helpers against hand-derived cases (the semantics of
// pipeline/include/tensor.cuh:60-300: consecutive pieces, the empty piece {ptr, 1, 0}, the
// overlapping "+suffix" pieces used for indptr arrays, the rank split, the GEMM tag's layouts).
// Prints "ok" and exits 0, or names the first failing case.
#include <cstdio>
#include <cstdlib>

#include "tensor.h"

namespace nflog {
int level() { return OFF; }
void write(Level, const char*, ...) {}
}  // namespace nflog

#define CHECK(c) do { if (!(c)) { std::printf("FAILED %s:%d %s\n", __FILE__, __LINE__, #c); return 1; } } while (0)

int main() {
  int buf[64];
  for (int i = 0; i < 64; ++i) buf[i] = i;
  const auto ROW = PllmLayout::ROW_MAJOR;

  pllmTensor<int> t(buf, 8, 4, ROW);   // 8 rows of 4
  CHECK(t.size() == 32 && t.bytes() == 128 && t.dimC() == 4);
  auto s = t.subtensor(2, 3);
  CHECK(s.ptr == buf + 8 && s.dim1 == 3 && s.dim2 == 4);
  CHECK(t.subtensor(5).dim1 == 3 && t.subtensor(5).ptr == buf + 20);
  bool threw = false;
  try { t.subtensor(8, 0); } catch (const std::out_of_range&) { threw = true; }
  CHECK(threw);
  threw = false;
  try { t.subtensor(6, 3); } catch (const std::out_of_range&) { threw = true; }
  CHECK(threw);
  CHECK(t.sameDirection(PllmDimension::ROW) && !t.sameDirection(PllmDimension::COLUMN));
  CHECK(pllmTensor<int>(buf, 2, 2, PllmLayout::COL_MAJOR).sameDirection(PllmDimension::COLUMN));
  CHECK(t.checkShape(pllmTensor<int>(buf + 1, 8, 4, ROW)) && !t.checkShape(pllmTensor<int>(buf, 4, 8, ROW)));
  CHECK(!t.assertShape(pllmTensor<int>(buf, 8, 4, PllmLayout::COL_MAJOR)));
  CHECK(t.shapeString() == "[8x4 ROW_MAJOR]");

  // plain split 3 + 0 + 5: the empty piece has size 0 and sits where the next one starts
  auto p = t.splitTensor(PllmDimension::ROW, 3, 0, 5);
  CHECK(p[0].ptr == buf && p[0].dim1 == 3 && p[0].dim2 == 4);
  CHECK(p[1].size() == 0 && p[1].ptr == buf + 12 && p[1].dim1 == 1 && p[1].dim2 == 0);
  CHECK(p[2].ptr == buf + 12 && p[2].dim1 == 5);

  // indptr of 6 requests (7 entries) cut into 2 | 0 | 4 requests with one shared entry
  pllmTensor<int> ind(buf, size_t(7));
  uint32_t lens_arr[3] = {2, 0, 4};
  std::span<uint32_t, 3> lens(lens_arr, 3);
  auto q = ind.splitTensor(PllmDimension::ROW, lens, 1U);
  CHECK(q[0].ptr == buf && q[0].size() == 3);
  CHECK(q[1].ptr == buf + 2 && q[1].size() == 1);
  CHECK(q[2].ptr == buf + 2 && q[2].size() == 5);
  // suffix 0: an empty piece is the empty tensor
  pllmTensor<int> six(buf, size_t(6));
  auto r = six.splitTensor(PllmDimension::ROW, lens);
  CHECK(r[0].size() == 2 && r[1].size() == 0 && r[1].dim2 == 0 && r[2].size() == 4 && r[2].ptr == buf + 2);
  // per-piece suffix {1, 2, 1}: the middle piece sees one entry more
  uint32_t suf_arr[3] = {1, 2, 1};
  std::span<uint32_t, 3> suf(suf_arr, 3);
  auto u = ind.splitTensor(PllmDimension::ROW, lens, suf);
  CHECK(u[0].size() == 3 && u[1].ptr == buf + 2 && u[1].size() == 2 && u[2].ptr == buf + 2 && u[2].size() == 5);

  // rank split: 10 rows over 4 ranks = 2, 2, 2, 4
  pllmTensor<int> ten(buf, 10, 2, ROW);
  CHECK(ten.getSubTensor(0, 4, PllmDimension::ROW).dim1 == 2);
  CHECK(ten.getSubTensor(2, 4, PllmDimension::ROW).ptr == buf + 8);
  CHECK(ten.getSubTensor(3, 4, PllmDimension::ROW).dim1 == 4 && ten.getSubTensor(3, 4, PllmDimension::ROW).ptr == buf + 12);
  CHECK(t.slice(PllmDimension::ROW, 1, 4).dim1 == 3 && t.slice(PllmDimension::ROW, 1, 4).ptr == buf + 4);

  auto c = tensor_cast<int, unsigned>(t);
  CHECK((void*)c.ptr == (void*)buf && c.dim1 == 8 && c.dim2 == 4);

  const std::string tag = "128_256_32_64_64_32_1_3_RowMajor_ColumnMajor_RowMajor";
  CHECK(getMajorType(tag, 0) == PllmLayout::ROW_MAJOR);
  CHECK(getMajorType(tag, 1) == PllmLayout::COL_MAJOR);
  CHECK(getMajorType(tag, 2) == PllmLayout::ROW_MAJOR);
  threw = false;
  try { getMajorType(tag, 3); } catch (const std::out_of_range&) { threw = true; }
  CHECK(threw);
  threw = false;
  try { getMajorType("128_256_RowMajor_Sideways_RowMajor", 1); } catch (const std::invalid_argument&) { threw = true; }
  CHECK(threw);
  threw = false;
  try { getMajorType("RowMajor", 0); } catch (const std::invalid_argument&) { threw = true; }
  CHECK(threw);
  std::printf("ok\n");
  return 0;
}
