// Host-side check of the in-register transform algebra of fbcuda_amd/csrc/fft_regs.h:
// the header holds no device intrinsics, so a host compiler can run the very templates
// the kernels instantiate.  Compared with a naive fp64 DFT:
//   * regFFT<N, forward / inverse> for N = 2 ... 128 (output index slot<N>(k)),
//   * the real-input fix-up: Z = FFT of the even/odd packing -> F[0 .. H] of the real
//     2H-point transform (realFixupForward), and its inverse (realFixupInverse, gain 2).
// Prints OK and returns 0 when every relative L2 error is below 1e-6.
#include <cmath>
#include <cstdio>
#include <vector>

#include "../../fbcuda_amd/csrc/fft_regs.h"

using fbfft_amd::c32;

static unsigned long long state = 0x9e3779b97f4a7c15ull;
static float nextFloat() {
  state = state * 6364136223846793005ull + 1442695040888963407ull;
  return (float)((double)(state >> 40) / (double)(1ull << 24)) * 2.0f - 1.0f;
}

static int failures = 0;
static void expectClose(const char* what, int n, double err2, double ref2) {
  const double rel = std::sqrt(err2 / (ref2 > 0 ? ref2 : 1));
  if (!(rel < 1e-6)) {
    std::printf("FAIL %s N=%d rel-L2 %.3e\n", what, n, rel);
    ++failures;
  }
}

template <int N, bool FWD>
static void checkComplex() {
  c32 a[N];
  std::vector<double> xr(N), xi(N);
  for (int n = 0; n < N; ++n) {
    a[n] = c32{nextFloat(), nextFloat()};
    xr[n] = a[n].x;
    xi[n] = a[n].y;
  }
  fbfft_amd::regFFT<N, FWD>(a);
  const double sign = FWD ? -1.0 : 1.0;
  double err2 = 0, ref2 = 0;
  for (int k = 0; k < N; ++k) {
    double re = 0, im = 0;
    for (int n = 0; n < N; ++n) {
      const double ang = sign * 2.0 * M_PI * (double)((k * n) % N) / N;
      re += xr[n] * std::cos(ang) - xi[n] * std::sin(ang);
      im += xr[n] * std::sin(ang) + xi[n] * std::cos(ang);
    }
    const c32 got = a[fbfft_amd::slot<N>(k)];
    err2 += (got.x - re) * (got.x - re) + (got.y - im) * (got.y - im);
    ref2 += re * re + im * im;
  }
  expectClose(FWD ? "regFFT forward" : "regFFT inverse", N, err2, ref2);
}

// real transform of 2H points through the H-point complex transform and the fix-ups
template <int H>
static void checkReal() {
  constexpr int N = 2 * H;
  std::vector<double> x(N);
  c32 z[H];
  for (int j = 0; j < H; ++j) {
    z[j] = c32{nextFloat(), nextFloat()};
    x[2 * j] = z[j].x;
    x[2 * j + 1] = z[j].y;
  }
  fbfft_amd::regFFT<H, true>(z);
  c32 f[H];  // f[0] = (F[0], F[H]) packed, f[k] = F[k]
  fbfft_amd::realFixupForward<H>(z, f);
  double err2 = 0, ref2 = 0;
  for (int k = 0; k <= H; ++k) {
    double re = 0, im = 0;
    for (int n = 0; n < N; ++n) {
      const double ang = -2.0 * M_PI * (double)((k * n) % N) / N;
      re += x[n] * std::cos(ang);
      im += x[n] * std::sin(ang);
    }
    double gr, gi;
    if (k == 0) { gr = f[0].x; gi = 0; }
    else if (k == H) { gr = f[0].y; gi = 0; }
    else { gr = f[k].x; gi = f[k].y; }
    err2 += (gr - re) * (gr - re) + (gi - im) * (gi - im);
    ref2 += re * re + im * im;
  }
  expectClose("real fix-up forward", N, err2, ref2);
  // and back: fix-up (gain 2), inverse H-point transform (gain H): x * 2H
  c32 w[H];
  fbfft_amd::realFixupInverse<H>(f, w);
  fbfft_amd::regFFT<H, false>(w);
  err2 = ref2 = 0;
  for (int j = 0; j < H; ++j) {
    const c32 got = w[fbfft_amd::slot<H>(j)];
    const double e0 = got.x - N * x[2 * j], e1 = got.y - N * x[2 * j + 1];
    err2 += e0 * e0 + e1 * e1;
    ref2 += (double)N * N * (x[2 * j] * x[2 * j] + x[2 * j + 1] * x[2 * j + 1]);
  }
  expectClose("real fix-up round trip", N, err2, ref2);
}

int main() {
  checkComplex<2, true>(); checkComplex<2, false>();
  checkComplex<4, true>(); checkComplex<4, false>();
  checkComplex<8, true>(); checkComplex<8, false>();
  checkComplex<16, true>(); checkComplex<16, false>();
  checkComplex<32, true>(); checkComplex<32, false>();
  checkComplex<64, true>(); checkComplex<64, false>();
  checkComplex<128, true>(); checkComplex<128, false>();
  checkReal<2>(); checkReal<4>(); checkReal<8>(); checkReal<16>(); checkReal<32>(); checkReal<64>();
  if (failures) return 1;
  std::printf("OK\n");
  return 0;
}
