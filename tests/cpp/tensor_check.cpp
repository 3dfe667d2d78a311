// Host-only check of the facade's DeviceTensor and Complex (no GPU, no HIP runtime):
// the size / stride arithmetic external callers use to build operands, e.g.
// flattening [batch][planes][h][w] before fbfft2D<1>.  Expected values are written
// out by hand from the documented meaning of each operation.  Prints "OK".
#include <cmath>
#include <cstdio>
#include <stdexcept>

#include "cuda/Complex.cuh"
#include "cuda/DeviceTensor.cuh"

using namespace facebook::cuda;

static int failures = 0;
#define CHECK(cond) do { if (!(cond)) { std::printf("FAILED line %d: %s\n", __LINE__, #cond); ++failures; } } while (0)

template <typename F>
static bool throwsInvalid(F&& f) {
  try { f(); } catch (const std::invalid_argument&) { return true; }
  return false;
}

int main() {
  float* base = reinterpret_cast<float*>(0x1000);
  int sz[4] = {2, 3, 5, 7};
  DeviceTensor<float, 4> t(base, sz);
  CHECK(t.getStride(0) == 105 && t.getStride(1) == 35 && t.getStride(2) == 7 && t.getStride(3) == 1);
  CHECK(t.numElements() == 210 && t.isContiguous() && t.isConsistentlySized());
  CHECK(t.toString() == "sizes: [2, 3, 5, 7]  strides: [105, 35, 7, 1]");
  for (int i = 0; i < 4; ++i) CHECK(t.isContiguousDim(i));

  // flatten batch x planes, as callers do before the 2D transforms
  DeviceTensor<float, 3> flat = t.downcastOuter<3>();
  CHECK(flat.getSize(0) == 6 && flat.getSize(1) == 5 && flat.getSize(2) == 7);
  CHECK(flat.getStride(0) == 35 && flat.getStride(1) == 7 && flat.getStride(2) == 1 && flat.data() == base);
  DeviceTensor<float, 2> rows = t.downcastOuter<2>();
  CHECK(rows.getSize(0) == 30 && rows.getSize(1) == 7 && rows.getStride(0) == 7);
  DeviceTensor<float, 2> inner = t.downcastInner<2>();
  CHECK(inner.getSize(0) == 2 && inner.getSize(1) == 105 && inner.getStride(0) == 105 && inner.getStride(1) == 1);

  // padded rows: stride 8 for 7 columns
  int st[4] = {120, 40, 8, 1};
  DeviceTensor<float, 4> padded(base, sz, st);
  CHECK(!padded.isContiguous() && padded.isConsistentlySized());
  CHECK(padded.isContiguousDim(0) && padded.isContiguousDim(1) && !padded.isContiguousDim(2));
  CHECK(padded.downcastOuter<2>().getSize(0) == 30 && padded.downcastOuter<2>().getStride(0) == 8);
  CHECK(throwsInvalid([&] { padded.downcastInner<2>(); }));
  CHECK(throwsInvalid([&] { padded.downcastOuter<1>(); }));
  CHECK(!t.isSameSizeAndStride(padded) && t.isSameSize(padded) && t.isSameSizeAndStride(t));
  CHECK(!t.isSameSize(flat));

  // transpose swaps sizes and strides only
  DeviceTensor<float, 4> tr = t.transpose(1, 3);
  CHECK(tr.getSize(1) == 7 && tr.getSize(3) == 3 && tr.getStride(1) == 1 && tr.getStride(3) == 35);
  CHECK(!tr.isContiguous() && !tr.isConsistentlySized() && tr.data() == base);
  CHECK(throwsInvalid([&] { t.transpose(0, 4); }) && throwsInvalid([&] { t.transpose(-1, 0); }));

  // permuteDims reorders the sizes and recomputes dense strides
  DeviceTensor<float, 4> p = t;
  p.permuteDims({3, 0, 2, 1});
  CHECK(p.getSize(0) == 7 && p.getSize(1) == 2 && p.getSize(2) == 5 && p.getSize(3) == 3);
  CHECK(p.getStride(0) == 30 && p.getStride(1) == 15 && p.getStride(2) == 3 && p.getStride(3) == 1);
  CHECK(throwsInvalid([&] { DeviceTensor<float, 4> q = padded; q.permuteDims({0, 1, 2, 3}); }));
  CHECK(throwsInvalid([&] { DeviceTensor<float, 4> q = t; q.permuteDims({0, 1}); }));

  // upcasts
  DeviceTensor<float, 5> up = flat.upcastOuter<5>();
  CHECK(up.getSize(0) == 1 && up.getSize(1) == 1 && up.getSize(2) == 6 && up.getStride(0) == 210 && up.getStride(1) == 210);
  DeviceTensor<float, 5> ui = flat.upcastInner<5>();
  CHECK(ui.getSize(3) == 1 && ui.getSize(4) == 1 && ui.getStride(3) == 1 && ui.getSize(2) == 7 && ui.getStride(0) == 35);

  // views and indexing
  DeviceTensor<float, 2> plane = t.view<2>(t[1][2].data());
  CHECK(plane.data() == base + 105 + 70 && plane.getSize(0) == 5 && plane.getSize(1) == 7 && plane.getStride(0) == 7);
  CHECK(t.view<3>().data() == base && t.view<3>().getSize(0) == 3);
  CHECK(t[1][2][3][4].data() == base + 105 + 70 + 21 + 4);
  CHECK(padded[0][1][2].data() == base + 40 + 16);

  // cast: complex-as-float pairs seen as Complex keep sizes and strides
  int cs[3] = {4, 17, 32};
  DeviceTensor<Complex, 3> spec(reinterpret_cast<Complex*>(base), cs);
  struct Pair { float a, b; };
  DeviceTensor<Pair, 3> same = spec.cast<Pair>();
  CHECK(same.getSize(1) == 17 && same.getStride(0) == 17 * 32 && (void*)same.data() == (void*)base);

  // size-1 dimensions do not break contiguity
  int one[3] = {4, 1, 6}, oneSt[3] = {6, 999, 1};
  CHECK((DeviceTensor<float, 3>(base, one, oneSt).isContiguous()));
  int neg[2] = {3, 4}, negSt[2] = {4, 0};
  CHECK(!(DeviceTensor<float, 2>(base, neg, negSt).isConsistentlySized()));

  // Complex arithmetic (cuComplex.h definitions)
  Complex a(1.5f, -2.0f), b(0.25f, 4.0f);
  CHECK((a + b) == Complex(1.75f, 2.0f) && (a - b) == Complex(1.25f, -6.0f) && (-a) == Complex(-1.5f, 2.0f));
  CHECK((a * b) == Complex(1.5f * 0.25f - (-2.0f) * 4.0f, 1.5f * 4.0f + (-2.0f) * 0.25f));
  Complex q = a / b;  // (a * conj b) / |b|^2 = (-7.625 - 6.5 i) / 16.0625
  CHECK(std::fabs(q.re() - (-7.625f / 16.0625f)) < 1e-6f && std::fabs(q.im() - (-6.5f / 16.0625f)) < 1e-6f);
  Complex big(3e30f, 4e30f);  // the scaled division does not overflow where |b|^2 would
  Complex r = big / big;
  CHECK(std::fabs(r.re() - 1.0f) < 1e-6f && std::fabs(r.im()) < 1e-6f);
  CHECK(a.conjugate() == Complex(1.5f, 2.0f) && a.transpose() == Complex(-2.0f, 1.5f) && a != b);
  Complex acc = a;
  acc += b; acc -= a; acc *= a; acc /= a;
  CHECK(std::fabs(acc.re() - b.re()) < 1e-6f && std::fabs(acc.im() - b.im()) < 1e-6f);
  Complex e;
  e.cexp(0.5f);
  CHECK(std::fabs(e.re() - std::cos(0.5f)) < 1e-7f && std::fabs(e.im() - std::sin(0.5f)) < 1e-7f);
  CHECK(Complex(2.0f) == Complex(2.0f, 0.0f) && Complex() == Complex(0.0f, 0.0f));

  if (failures) return 1;
  std::printf("OK\n");
  return 0;
}
