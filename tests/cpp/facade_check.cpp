// Exercises the C++ facade exactly as host code written against fbcuda's headers
// would: DeviceTensor views, fbfft2D<1> / fbifft2D<1>, transposeMM and
// FBFFTParameters, on device buffers from the HIP runtime.  Prints "OK" and
// returns 0 when every check is within tolerance.
#include <hip/hip_runtime_api.h>

#include <cmath>
#include <cstdio>
#include <vector>

#include "cuda/fbfft/FBFFT.cuh"
#include "cuda/MM.cuh"
#include "cuda/fbfft/FFTIteratedConvolution.cuh"

using namespace facebook::cuda;
using facebook::cuda::fbfft::FBFFTParameters;

#define HIP_OK(x) do { if ((x) != hipSuccess) { std::printf("HIP error at %d\n", __LINE__); return 2; } } while (0)

int main() {
  const int B = 3, N = 32, nc = N / 2 + 1;
  std::vector<float> x((size_t)B * N * N);
  unsigned s = 12345u;
  for (auto& v : x) { s = s * 1664525u + 1013904223u; v = (float)(s >> 8) / 8388608.0f - 1.0f; }

  float *dx, *dspec, *dback;
  HIP_OK(hipMalloc((void**)&dx, x.size() * 4));
  HIP_OK(hipMalloc((void**)&dspec, (size_t)B * nc * N * 2 * 4));
  HIP_OK(hipMalloc((void**)&dback, x.size() * 4));
  HIP_OK(hipMemcpy(dx, x.data(), x.size() * 4, hipMemcpyHostToDevice));

  int rs[3] = {B, N, N}, cs[4] = {B, nc, N, 2};
  DeviceTensor<float, 3> real(dx, rs), back(dback, rs);
  DeviceTensor<float, 4> spec(dspec, cs);
  if (fbfft::fbfft2D<1>(real, spec) != FBFFTParameters::Success) return 3;
  int ccs[3] = {B, nc, N};
  DeviceTensor<Complex, 3> cspec(reinterpret_cast<Complex*>(dspec), ccs);
  if (fbfft::fbifft2D<1>(cspec, back) != FBFFTParameters::Success) return 4;
  HIP_OK(hipDeviceSynchronize());

  std::vector<float> spec_h((size_t)B * nc * N * 2), back_h(x.size());
  HIP_OK(hipMemcpy(spec_h.data(), dspec, spec_h.size() * 4, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(back_h.data(), dback, back_h.size() * 4, hipMemcpyDeviceToHost));

  // spectrum against a literal double DFT of plane 1: out[b][ky][kx], ky <= N/2
  double num = 0, den = 0;
  const int b = 1;
  for (int ky = 0; ky < nc; ++ky)
    for (int kx = 0; kx < N; ++kx) {
      double re = 0, im = 0;
      for (int y = 0; y < N; ++y)
        for (int xx = 0; xx < N; ++xx) {
          double a = -2.0 * M_PI * ((ky * y + kx * xx) % N) / N;
          re += x[((size_t)b * N + y) * N + xx] * std::cos(a);
          im += x[((size_t)b * N + y) * N + xx] * std::sin(a);
        }
      size_t i = (((size_t)b * nc + ky) * N + kx) * 2;
      num += (spec_h[i] - re) * (spec_h[i] - re) + (spec_h[i + 1] - im) * (spec_h[i + 1] - im);
      den += re * re + im * im;
    }
  const double e1 = std::sqrt(num / den);
  num = den = 0;
  for (size_t i = 0; i < x.size(); ++i) {
    double d = back_h[i] / (double)(N * N) - x[i];
    num += d * d;
    den += (double)x[i] * x[i];
  }
  const double e2 = std::sqrt(num / den);

  // unsupported size through the facade
  int bad[4] = {B, 129, 256, 2};
  DeviceTensor<float, 4> badSpec(dspec, bad);
  const bool e3 = fbfft::fbfft2D<1>(real, badSpec) == FBFFTParameters::UnsupportedSize;

  FBFFTParameters p;
  p.inverse().withPadLeft(2).withPadUp(1).normalize(true);
  const bool e4 = p.inverseFFT() && p.padLeft() == 2 && p.padUp() == 1 && p.normalizeFFT();

  std::printf("fbfft2D rel-L2 vs double DFT %.3e, round trip %.3e, errors %d, params %d\n", e1, e2,
              (int)e3, (int)e4);
  hipFree(dx); hipFree(dspec); hipFree(dback);
  if (e1 < 1e-5 && e2 < 1e-5 && e3 && e4) { std::printf("OK\n"); return 0; }
  return 1;
}
