// 2D real-to-complex / complex-to-real transforms of 2x2 and 4x4 planes (replaces
// decimateInFrequencyHermitian2DWarpKernel, fbfft/FBFFT2D-inl.cuh:124-222, and
// decimateInFrequencyInverseHermitian2DWarpKernel, fbfft/FBIFFT2D-inl.cuh:188-247,
// for the two sizes that reach them: dispatch at FBFFT2D-inl.cuh:611-612 and
// FBIFFT2D-inl.cuh:684-712).
//
// A plane is 16 or 64 bytes, so one lane transforms a whole plane in VGPRs: N
// row transforms, then N/2+1 column transforms, all with the trivial twiddles
// 1 and -i.  Spectrum layout is the warp kernel's: cplx[b][kx][ky] with the
// horizontal frequency halved (store2D, FBFFT2D-inl.cuh:71-85).  The reference
// carries two planes as the real and imaginary part of one complex transform;
// here planes are independent, which gives the same values up to rounding on
// Hermitian input and needs no even batch.
#include "common.h"
#include "fft_regs.h"

namespace fbfft_amd {
namespace {

constexpr int kTinyThreads = 256;

template <int N>
__global__ __launch_bounds__(kTinyThreads) void fft2dTinyForward(RealView in, CplxView out, int padL,
                                                                 int padU) {
  const int b = blockIdx.x * kTinyThreads + threadIdx.x;
  if (b >= in.B) return;
  const float* src = in.data + (size_t)b * in.sb;
  c32 rows[N][N];
  staticFor<N>([&](auto yy) {
    constexpr int y = decltype(yy)::value;
    staticFor<N>([&](auto xx) {
      constexpr int x = decltype(xx)::value;
      const bool inside = inWindow(y, x, padU, padL, in.h, in.w);
      rows[y][x] = c32{inside ? src[(size_t)(y - padU) * in.sy + (size_t)(x - padL) * in.sx] : 0.0f,
                       0.0f};
    });
    difFFT<N, true>(rows[y]);
  });
  float* dst = out.data + (size_t)b * out.sb;
  staticFor<N / 2 + 1>([&](auto kk) {
    constexpr int kx = decltype(kk)::value;
    c32 col[N];
    staticFor<N>([&](auto yy) {
      constexpr int y = decltype(yy)::value;
      col[y] = rows[y][slot<N>(kx)];
    });
    difFFT<N, true>(col);
    staticFor<N>([&](auto ff) {
      constexpr int ky = decltype(ff)::value;
      *reinterpret_cast<float2*>(dst + (size_t)kx * out.sr + (size_t)ky * out.sc) = col[slot<N>(ky)];
    });
  });
}

template <int N>
__global__ __launch_bounds__(kTinyThreads) void fft2dTinyInverse(CplxView in, RealView out, int padL,
                                                                 int padU) {
  const int b = blockIdx.x * kTinyThreads + threadIdx.x;
  if (b >= in.B) return;
  const float* src = in.data + (size_t)b * in.sb;
  // g[kx][y]: inverse transform along ky of the N/2+1 stored kx
  c32 g[N / 2 + 1][N];
  staticFor<N / 2 + 1>([&](auto kk) {
    constexpr int kx = decltype(kk)::value;
    c32 col[N];
    staticFor<N>([&](auto ff) {
      constexpr int ky = decltype(ff)::value;
      col[ky] = *reinterpret_cast<const float2*>(src + (size_t)kx * in.sr + (size_t)ky * in.sc);
    });
    difFFT<N, false>(col);
    staticFor<N>([&](auto yy) {
      constexpr int y = decltype(yy)::value;
      g[kx][y] = col[slot<N>(y)];
    });
  });
  float* dst = out.data + (size_t)b * out.sb;
  staticFor<N>([&](auto yy) {
    constexpr int y = decltype(yy)::value;
    // Hermitian extension along kx (the expansion of load2D, FBIFFT2D-inl.cuh:42-57)
    c32 row[N];
    staticFor<N>([&](auto kk) {
      constexpr int kx = decltype(kk)::value;
      if constexpr (kx <= N / 2)
        row[kx] = g[kx][y];
      else
        row[kx] = cconj(g[N - kx][y]);
    });
    difFFT<N, false>(row);
    staticFor<N>([&](auto xx) {
      constexpr int x = decltype(xx)::value;
      if (inWindow(y, x, padU, padL, out.h, out.w))
        dst[(size_t)(y - padU) * out.sy + (size_t)(x - padL) * out.sx] = row[slot<N>(x)].x;
    });
  });
}

}  // namespace

int launchFft2dTinyForward(int N, const RealView& real, const CplxView& cplx, int padL, int padU,
                           hipStream_t s) {
  dim3 grid(ceilDiv(real.B, kTinyThreads)), block(kTinyThreads);
  if (N == 2)
    fft2dTinyForward<2><<<grid, block, 0, s>>>(real, cplx, padL, padU);
  else if (N == 4)
    fft2dTinyForward<4><<<grid, block, 0, s>>>(real, cplx, padL, padU);
  else
    return FBFFT_UNSUPPORTED_SIZE;
  return launchStatus();
}

int launchFft2dTinyInverse(int N, const CplxView& cplx, const RealView& real, int padL, int padU,
                           hipStream_t s) {
  dim3 grid(ceilDiv(real.B, kTinyThreads)), block(kTinyThreads);
  if (N == 2)
    fft2dTinyInverse<2><<<grid, block, 0, s>>>(cplx, real, padL, padU);
  else if (N == 4)
    fft2dTinyInverse<4><<<grid, block, 0, s>>>(cplx, real, padL, padU);
  else
    return FBFFT_UNSUPPORTED_SIZE;
  return launchStatus();
}

}  // namespace fbfft_amd
