// Exercises the C++ facade exactly as host code written against fbcuda's headers
// would: DeviceTensor views, fbfft2D<1> / fbifft2D<1>, FBFFTParameters, the
// three passes of the convolution layer and the tiled FFTIteratedConvolution
// with host-built descriptors, on device buffers from the HIP runtime.  Prints
// "OK" and returns 0 when every check is within tolerance.
#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <vector>

#include "cuda/fbfft/FBFFT.cuh"
#include "cuda/MM.cuh"
#include "cuda/fbfft/FFTIteratedConvolution.cuh"
#include "cuda/fbfft/FBFFTCommon.cuh"
#include "cuda/MemoryAccess.cuh"

using namespace facebook::cuda;
using facebook::cuda::fbfft::FBFFTParameters;

#define HIP_OK(x) do { if ((x) != hipSuccess) { std::printf("HIP error at %d\n", __LINE__); return 2; } } while (0)

namespace {

struct Lcg {
  unsigned s;
  float next() { s = s * 1664525u + 1013904223u; return (float)(s >> 8) / 8388608.0f - 1.0f; }
};

double relL2(const std::vector<float>& got, const std::vector<double>& want) {
  double num = 0, den = 0;
  for (size_t i = 0; i < want.size(); ++i) {
    num += (got[i] - want[i]) * (got[i] - want[i]);
    den += want[i] * want[i];
  }
  return std::sqrt(num / den);
}

template <typename T>
T* upload(const std::vector<T>& h) {
  T* d = nullptr;
  if (hipMalloc((void**)&d, h.size() * sizeof(T)) != hipSuccess) return nullptr;
  hipMemcpy(d, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice);
  return d;
}

std::vector<float> download(const float* d, size_t n) {
  std::vector<float> h(n);
  hipMemcpy(h.data(), d, n * 4, hipMemcpyDeviceToHost);
  return h;
}

// The convolution layer through the facade against literal double loops.
// Returns the largest relative error of the four results (three passes on the
// split path, forward pass on the tiled path).
double convLayerError() {
  const int B = 2, Ci = 3, Co = 4, H = 21, W = 19, k = 3, N = 16;
  const int oH = H - k + 1, oW = W - k + 1;
  Lcg g{777u};
  std::vector<float> x((size_t)B * Ci * H * W), w((size_t)Co * Ci * k * k), go((size_t)B * Co * oH * oW);
  for (auto& v : x) v = g.next();
  for (auto& v : w) v = 0.1f * g.next();
  for (auto& v : go) v = g.next();
  auto X = [&](int b, int c, int y, int xx) { return (double)x[(((size_t)b * Ci + c) * H + y) * W + xx]; };
  auto Wt = [&](int f, int c, int u, int v) { return (double)w[(((size_t)f * Ci + c) * k + u) * k + v]; };
  auto G = [&](int b, int f, int y, int xx) { return (double)go[(((size_t)b * Co + f) * oH + y) * oW + xx]; };
  std::vector<double> out((size_t)B * Co * oH * oW, 0.0), gi(x.size(), 0.0), gw(w.size(), 0.0);
  for (int b = 0; b < B; ++b)
    for (int f = 0; f < Co; ++f)
      for (int c = 0; c < Ci; ++c)
        for (int y = 0; y < oH; ++y)
          for (int xx = 0; xx < oW; ++xx)
            for (int u = 0; u < k; ++u)
              for (int v = 0; v < k; ++v) {
                out[(((size_t)b * Co + f) * oH + y) * oW + xx] += X(b, c, y + u, xx + v) * Wt(f, c, u, v);
                gi[(((size_t)b * Ci + c) * H + y + u) * W + xx + v] += G(b, f, y, xx) * Wt(f, c, u, v);
                gw[(((size_t)f * Ci + c) * k + u) * k + v] += X(b, c, y + u, xx + v) * G(b, f, y, xx);
              }

  float *dx = upload(x), *dw = upload(w), *dgo = upload(go);
  float *dout, *dgi, *dgw, *dtiled;
  hipMalloc((void**)&dout, out.size() * 4);
  hipMalloc((void**)&dtiled, out.size() * 4);
  hipMalloc((void**)&dgi, gi.size() * 4);
  hipMalloc((void**)&dgw, gw.size() * 4);
  int xs[4] = {B, Ci, H, W}, wsz[4] = {Co, Ci, k, k}, os[4] = {B, Co, oH, oW};
  DeviceTensor<float, 4> tx(dx, xs), tw(dw, wsz), tgo(dgo, os), tout(dout, os), tgi(dgi, xs),
      tgw(dgw, wsz), ttiled(dtiled, os);
  double worst = 0;

  // split path needs the whole plane inside one FFT: run it on the top-left 16 x 16 window
  {
    const int h = 16, ww = 16, ph = h - k + 1, pw = ww - k + 1;
    int xv[4] = {B, Ci, h, ww}, ov[4] = {B, Co, ph, pw};
    int xst[4] = {Ci * H * W, H * W, W, 1}, ost[4] = {Co * oH * oW, oH * oW, oW, 1};
    DeviceTensor<float, 4> vx(dx, xv, xst), vgo(dgo, ov, ost), vout(dout, ov, ost), vgi(dgi, xv, xst);
    using Pass = fbfft::detail::FFTConvolutionPassFFI;
    size_t bytes = 0;
    for (int p = 0; p < 3; ++p) {
      Pass pass;
      pass.pass = p;
      bytes = std::max(bytes, fbfft::fftConvolutionWorkspace(pass, B, Ci, Co, N));
    }
    void* ws;
    hipMalloc(&ws, bytes);
    hipMemset(dout, 0, out.size() * 4);
    hipMemset(dgi, 0, gi.size() * 4);
    if (fbfft::fftConvolutionUpdateOutput(vx, tw, vout, N, ws, bytes) != FBFFTParameters::Success) return 1;
    if (fbfft::fftConvolutionUpdateGradInput(vgo, tw, vgi, N, ws, bytes) != FBFFTParameters::Success) return 1;
    if (fbfft::fftConvolutionAccGradParameters(vx, vgo, tgw, N, 1.0f, false, ws, bytes) !=
        FBFFTParameters::Success)
      return 1;
    hipDeviceSynchronize();
    // the same three quantities restricted to the window, in double
    std::vector<double> o2((size_t)B * Co * ph * pw, 0.0), gi2((size_t)B * Ci * h * ww, 0.0), gw2(w.size(), 0.0);
    for (int b = 0; b < B; ++b)
      for (int f = 0; f < Co; ++f)
        for (int c = 0; c < Ci; ++c)
          for (int y = 0; y < ph; ++y)
            for (int xx = 0; xx < pw; ++xx)
              for (int u = 0; u < k; ++u)
                for (int v = 0; v < k; ++v) {
                  o2[(((size_t)b * Co + f) * ph + y) * pw + xx] += X(b, c, y + u, xx + v) * Wt(f, c, u, v);
                  gi2[(((size_t)b * Ci + c) * h + y + u) * ww + xx + v] += G(b, f, y, xx) * Wt(f, c, u, v);
                  gw2[(((size_t)f * Ci + c) * k + u) * k + v] += X(b, c, y + u, xx + v) * G(b, f, y, xx);
                }
    auto ho = download(dout, out.size()), hgi = download(dgi, gi.size()), hgw = download(dgw, gw.size());
    std::vector<float> co(o2.size()), cgi(gi2.size());
    for (int b = 0; b < B; ++b)
      for (int f = 0; f < Co; ++f)
        for (int y = 0; y < ph; ++y)
          for (int xx = 0; xx < pw; ++xx)
            co[(((size_t)b * Co + f) * ph + y) * pw + xx] = ho[(((size_t)b * Co + f) * oH + y) * oW + xx];
    for (int b = 0; b < B; ++b)
      for (int c = 0; c < Ci; ++c)
        for (int y = 0; y < h; ++y)
          for (int xx = 0; xx < ww; ++xx)
            cgi[(((size_t)b * Ci + c) * h + y) * ww + xx] = hgi[(((size_t)b * Ci + c) * H + y) * W + xx];
    worst = std::max(worst, relL2(co, o2));
    worst = std::max(worst, relL2(cgi, gi2));
    worst = std::max(worst, relL2(hgw, gw2));
    hipFree(ws);
  }

  // tiled path over the whole 21 x 19 image with host-built descriptors
  {
    using Tile = fbfft::detail::TiledDeviceTensor<float, 4>;
    const size_t n = fbfft::detail::makeTiles<N>(tx, ttiled, k, k, nullptr, nullptr, 0);
    if (n != 4) return 1;  // ceil(19/14) x ceil(17/14)
    std::vector<Tile> ins(n), outs(n);
    if (fbfft::detail::makeTiles<N>(tx, ttiled, k, k, ins.data(), outs.data(), n) != n) return 1;
    Tile *dins = upload(ins), *douts = upload(outs);
    fbfft::detail::FFTConvolutionPassFFI pass;
    pass.pass = fbfft::detail::FFTConvolutionPassFFI::FFT_UpdateOutput;
    if (!fbfft::detail::FFTIteratedConvolution<N>(dins, douts, tw, pass, 1.0f, B, n, 0)) return 1;
    hipDeviceSynchronize();
    worst = std::max(worst, relL2(download(dtiled, out.size()), out));
    // the same descriptors through a workspace
    HIP_OK(hipMemset(dtiled, 0xff, out.size() * 4));
    const size_t wsBytes = fbfft::detail::iteratedConvolutionWorkspace<N>(tw, pass, B, n);
    if (wsBytes == 0) return 1;
    void* ws;
    HIP_OK(hipMalloc(&ws, wsBytes));
    if (!fbfft::detail::FFTIteratedConvolution<N>(dins, douts, tw, pass, 1.0f, B, n, ws, wsBytes, 0))
      return 1;
    hipDeviceSynchronize();
    worst = std::max(worst, relL2(download(dtiled, out.size()), out));
    hipFree(ws);
    hipFree(dins);
    hipFree(douts);
  }
  hipFree(dx); hipFree(dw); hipFree(dgo); hipFree(dout); hipFree(dgi); hipFree(dgw); hipFree(dtiled);
  return worst;
}

}  // namespace

int main() {
  {  // host helpers of the reference's headers
    using namespace facebook::cuda;
    if (fbfft::numHermitian(32) != 17 || fbfft::numHermitian(2) != 2) return 1;
    int sz3[3] = {4, 5, 7};
    DeviceTensor<float, 3> t3(nullptr, sz3);
    if (!inBounds(2, 3, 2, 3, t3) || !inBounds(6, 9, 2, 3, t3) || inBounds(7, 3, 2, 3, t3) ||
        inBounds(1, 3, 2, 3, t3) || inBounds(2, 10, 2, 3, t3))
      return 1;
  }
  const int B = 3, N = 32, nc = N / 2 + 1;
  std::vector<float> x((size_t)B * N * N);
  unsigned s = 12345u;
  for (auto& v : x) { s = s * 1664525u + 1013904223u; v = (float)(s >> 8) / 8388608.0f - 1.0f; }

  float *dx, *dspec, *dback;
  HIP_OK(hipMalloc((void**)&dx, x.size() * 4));
  HIP_OK(hipMalloc((void**)&dspec, (size_t)B * nc * N * 2 * 4));
  HIP_OK(hipMalloc((void**)&dback, x.size() * 4));
  HIP_OK(hipMemcpy(dx, x.data(), x.size() * 4, hipMemcpyHostToDevice));

  // operands arrive as [batch][planes][h][w]; the callers flatten batch x planes with
  // downcastOuter before the 2D transforms
  int rs4[4] = {1, B, N, N}, cs5[5] = {1, B, nc, N, 2}, rs[3] = {B, N, N};
  DeviceTensor<float, 4> real4(dx, rs4);
  DeviceTensor<float, 5> spec5(dspec, cs5);
  DeviceTensor<float, 3> real = real4.downcastOuter<3>(), back(dback, rs);
  DeviceTensor<float, 4> spec = spec5.downcastOuter<4>();
  if (real.getSize(0) != B || spec.getSize(1) != nc || !real.isContiguous()) return 3;
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

  const double e5 = convLayerError();

  std::printf("fbfft2D rel-L2 vs double DFT %.3e, round trip %.3e, errors %d, params %d, "
              "convolution layer %.3e\n", e1, e2, (int)e3, (int)e4, e5);
  hipFree(dx); hipFree(dspec); hipFree(dback);
  if (e1 < 1e-5 && e2 < 1e-5 && e3 && e4 && e5 < 1e-4) { std::printf("OK\n"); return 0; }
  return 1;
}
