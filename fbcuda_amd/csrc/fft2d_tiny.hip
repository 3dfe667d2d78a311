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

// spec[kx][ky] of one real plane x[y][x], all in registers
template <int N>
__device__ __forceinline__ void forwardPlane(const float (&x)[N][N], c32 (&spec)[N / 2 + 1][N]) {
  c32 rows[N][N];
  staticFor<N>([&](auto yy) {
    constexpr int y = decltype(yy)::value;
    staticFor<N>([&](auto xx) { rows[y][decltype(xx)::value] = c32{x[y][decltype(xx)::value], 0.0f}; });
    regFFT<N, true>(rows[y]);
  });
  staticFor<N / 2 + 1>([&](auto kk) {
    constexpr int kx = decltype(kk)::value;
    c32 col[N];
    staticFor<N>([&](auto yy) {
      constexpr int y = decltype(yy)::value;
      col[y] = rows[y][slot<N>(kx)];
    });
    regFFT<N, true>(col);
    staticFor<N>([&](auto ff) {
      constexpr int ky = decltype(ff)::value;
      spec[kx][ky] = col[slot<N>(ky)];
    });
  });
}

// x[y][x] * N*N from spec[kx][ky], kx = 0..N/2
template <int N>
__device__ __forceinline__ void inversePlane(const c32 (&spec)[N / 2 + 1][N], float (&x)[N][N]) {
  // g[kx][y]: inverse transform along ky of the N/2+1 stored kx
  c32 g[N / 2 + 1][N];
  staticFor<N / 2 + 1>([&](auto kk) {
    constexpr int kx = decltype(kk)::value;
    c32 col[N];
    staticFor<N>([&](auto ff) { col[decltype(ff)::value] = spec[kx][decltype(ff)::value]; });
    regFFT<N, false>(col);
    staticFor<N>([&](auto yy) {
      constexpr int y = decltype(yy)::value;
      g[kx][y] = col[slot<N>(y)];
    });
  });
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
    regFFT<N, false>(row);
    staticFor<N>([&](auto xx) {
      constexpr int xi = decltype(xx)::value;
      x[y][xi] = row[slot<N>(xi)].x;
    });
  });
}

template <int N>
__global__ __launch_bounds__(kTinyThreads) void fft2dTinyForward(RealView in, CplxView out, int padL,
                                                                 int padU) {
  const int b = blockIdx.x * kTinyThreads + threadIdx.x;
  if (b >= in.B) return;
  const float* src = in.data + (size_t)b * in.sb;
  float x[N][N];
  staticFor<N>([&](auto yy) {
    constexpr int y = decltype(yy)::value;
    staticFor<N>([&](auto xx) {
      constexpr int xi = decltype(xx)::value;
      const bool inside = inWindow(y, xi, padU, padL, in.h, in.w);
      x[y][xi] = inside ? src[(size_t)(y - padU) * in.sy + (size_t)(xi - padL) * in.sx] : 0.0f;
    });
  });
  c32 spec[N / 2 + 1][N];
  forwardPlane<N>(x, spec);
  float* dst = out.data + (size_t)b * out.sb;
  staticFor<N / 2 + 1>([&](auto kk) {
    constexpr int kx = decltype(kk)::value;
    staticFor<N>([&](auto ff) {
      constexpr int ky = decltype(ff)::value;
      *reinterpret_cast<float2*>(dst + (size_t)kx * out.sr + (size_t)ky * out.sc) = spec[kx][ky];
    });
  });
}

template <int N>
__global__ __launch_bounds__(kTinyThreads) void fft2dTinyInverse(CplxView in, RealView out, int padL,
                                                                 int padU) {
  const int b = blockIdx.x * kTinyThreads + threadIdx.x;
  if (b >= in.B) return;
  const float* src = in.data + (size_t)b * in.sb;
  c32 spec[N / 2 + 1][N];
  staticFor<N / 2 + 1>([&](auto kk) {
    constexpr int kx = decltype(kk)::value;
    staticFor<N>([&](auto ff) {
      constexpr int ky = decltype(ff)::value;
      spec[kx][ky] = *reinterpret_cast<const float2*>(src + (size_t)kx * in.sr + (size_t)ky * in.sc);
    });
  });
  float x[N][N];
  inversePlane<N>(spec, x);
  float* dst = out.data + (size_t)b * out.sb;
  staticFor<N>([&](auto yy) {
    constexpr int y = decltype(yy)::value;
    staticFor<N>([&](auto xx) {
      constexpr int xi = decltype(xx)::value;
      if (inWindow(y, xi, padU, padL, out.h, out.w))
        dst[(size_t)(y - padU) * out.sy + (size_t)(xi - padL) * out.sx] = x[y][xi];
    });
  });
}

// Contiguous, 16-byte aligned batches: a lane's plane is 16 or 64 bytes and its
// spectrum 32 or 96, so lane-private global accesses would touch every cache line
// four or six times.  The workgroup moves its 256 planes between HBM and LDS as one
// 16-byte stream instead; in LDS a plane is padded so that the lanes' 16-byte reads
// and writes spread over the banks.
template <int N>
struct TinyCfg {
  static constexpr int IN = N * N;                  // floats per plane
  static constexpr int OUT = (N / 2 + 1) * N * 2;   // floats per spectrum
  static constexpr int INS = N == 4 ? 20 : 4;       // LDS strides (floats)
  static constexpr int OUTS = N == 4 ? 28 : 8;
  static constexpr int LDS = kTinyThreads * (INS > OUTS ? INS : OUTS);
};

// global (contiguous, PER floats per plane) <-> LDS (STRIDE floats per plane)
template <int PER, int STRIDE, bool TO_LDS>
__device__ __forceinline__ void moveTiny(float* global, float* stage, int planes, int t) {
  constexpr int Q = PER / 4;
  float v[4 * Q];  // plain floats: always promoted to registers
  float4* g4 = reinterpret_cast<float4*>(global);
  staticFor<Q>([&](auto ii) {
    constexpr int i = decltype(ii)::value;
    const int q = min(t + kTinyThreads * i, planes * Q - 1);  // tail lanes repeat the last word
    const float4 w = TO_LDS ? g4[q]
                            : *reinterpret_cast<const float4*>(stage + (q / Q) * STRIDE + 4 * (q % Q));
    v[4 * i] = w.x;
    v[4 * i + 1] = w.y;
    v[4 * i + 2] = w.z;
    v[4 * i + 3] = w.w;
  });
  staticFor<Q>([&](auto ii) {
    constexpr int i = decltype(ii)::value;
    const int q = t + kTinyThreads * i;
    if (q < planes * Q) {
      const float4 w = float4{v[4 * i], v[4 * i + 1], v[4 * i + 2], v[4 * i + 3]};
      if constexpr (TO_LDS)
        *reinterpret_cast<float4*>(stage + (q / Q) * STRIDE + 4 * (q % Q)) = w;
      else
        streamStore(g4 + q, w);
    }
  });
}

template <int N>
__global__ __launch_bounds__(kTinyThreads) void fft2dTinyForwardStream(const float* in, float* out,
                                                                       int B) {
  using C = TinyCfg<N>;
  __shared__ __align__(16) float stage[C::LDS];
  const int t = threadIdx.x;
  const int b0 = blockIdx.x * kTinyThreads;
  const int planes = min(kTinyThreads, B - b0);
  moveTiny<C::IN, C::INS, true>(const_cast<float*>(in) + (size_t)b0 * C::IN, stage, planes, t);
  __syncthreads();
  float x[N][N];
  staticFor<C::IN / 4>([&](auto ii) {
    constexpr int i = decltype(ii)::value;  // float4 i of the plane: floats 4i .. 4i+3
    const float4 v = *reinterpret_cast<const float4*>(stage + t * C::INS + 4 * i);
    x[(4 * i) / N][(4 * i) % N] = v.x;
    x[(4 * i + 1) / N][(4 * i + 1) % N] = v.y;
    x[(4 * i + 2) / N][(4 * i + 2) % N] = v.z;
    x[(4 * i + 3) / N][(4 * i + 3) % N] = v.w;
  });
  c32 spec[N / 2 + 1][N];
  forwardPlane<N>(x, spec);
  __syncthreads();  // every plane is in registers: the buffer takes the spectra
  staticFor<C::OUT / 4>([&](auto ii) {
    constexpr int i = decltype(ii)::value;  // complex 2i and 2i+1 of [kx][ky]
    const c32 a = spec[(2 * i) / N][(2 * i) % N], c = spec[(2 * i + 1) / N][(2 * i + 1) % N];
    *reinterpret_cast<float4*>(stage + t * C::OUTS + 4 * i) = float4{a.x, a.y, c.x, c.y};
  });
  __syncthreads();
  moveTiny<C::OUT, C::OUTS, false>(out + (size_t)b0 * C::OUT, stage, planes, t);
}

template <int N>
__global__ __launch_bounds__(kTinyThreads) void fft2dTinyInverseStream(const float* in, float* out,
                                                                       int B) {
  using C = TinyCfg<N>;
  __shared__ __align__(16) float stage[C::LDS];
  const int t = threadIdx.x;
  const int b0 = blockIdx.x * kTinyThreads;
  const int planes = min(kTinyThreads, B - b0);
  moveTiny<C::OUT, C::OUTS, true>(const_cast<float*>(in) + (size_t)b0 * C::OUT, stage, planes, t);
  __syncthreads();
  c32 spec[N / 2 + 1][N];
  staticFor<C::OUT / 4>([&](auto ii) {
    constexpr int i = decltype(ii)::value;
    const float4 v = *reinterpret_cast<const float4*>(stage + t * C::OUTS + 4 * i);
    spec[(2 * i) / N][(2 * i) % N] = c32{v.x, v.y};
    spec[(2 * i + 1) / N][(2 * i + 1) % N] = c32{v.z, v.w};
  });
  float x[N][N];
  inversePlane<N>(spec, x);
  __syncthreads();
  staticFor<C::IN / 4>([&](auto ii) {
    constexpr int i = decltype(ii)::value;
    *reinterpret_cast<float4*>(stage + t * C::INS + 4 * i) =
        float4{x[(4 * i) / N][(4 * i) % N], x[(4 * i + 1) / N][(4 * i + 1) % N],
               x[(4 * i + 2) / N][(4 * i + 2) % N], x[(4 * i + 3) / N][(4 * i + 3) % N]};
  });
  __syncthreads();
  moveTiny<C::IN, C::INS, false>(out + (size_t)b0 * C::IN, stage, planes, t);
}

bool streams(int N, const RealView& r, const CplxView& c, int padL, int padU) {
  return padL == 0 && padU == 0 && r.h == N && r.w == N && r.sx == 1 && r.sy == N &&
         r.sb == N * N && c.sc == 2 && c.sr == 2 * N && c.sb == (N / 2 + 1) * N * 2 &&
         aligned(r.data, 16) && aligned(c.data, 16);
}

}  // namespace

int launchFft2dTinyForward(int N, const RealView& real, const CplxView& cplx, int padL, int padU,
                           hipStream_t s) {
  dim3 grid(ceilDiv(real.B, kTinyThreads)), block(kTinyThreads);
  if (N != 2 && N != 4) return FBFFT_UNSUPPORTED_SIZE;
  if (streams(N, real, cplx, padL, padU)) {
    if (N == 2)
      fft2dTinyForwardStream<2><<<grid, block, 0, s>>>(real.data, cplx.data, real.B);
    else
      fft2dTinyForwardStream<4><<<grid, block, 0, s>>>(real.data, cplx.data, real.B);
  } else if (N == 2) {
    fft2dTinyForward<2><<<grid, block, 0, s>>>(real, cplx, padL, padU);
  } else {
    fft2dTinyForward<4><<<grid, block, 0, s>>>(real, cplx, padL, padU);
  }
  return launchStatus();
}

int launchFft2dTinyInverse(int N, const CplxView& cplx, const RealView& real, int padL, int padU,
                           hipStream_t s) {
  dim3 grid(ceilDiv(real.B, kTinyThreads)), block(kTinyThreads);
  if (N != 2 && N != 4) return FBFFT_UNSUPPORTED_SIZE;
  if (streams(N, real, cplx, padL, padU)) {
    if (N == 2)
      fft2dTinyInverseStream<2><<<grid, block, 0, s>>>(cplx.data, real.data, real.B);
    else
      fft2dTinyInverseStream<4><<<grid, block, 0, s>>>(cplx.data, real.data, real.B);
  } else if (N == 2) {
    fft2dTinyInverse<2><<<grid, block, 0, s>>>(cplx, real, padL, padU);
  } else {
    fft2dTinyInverse<4><<<grid, block, 0, s>>>(cplx, real, padL, padU);
  }
  return launchStatus();
}

}  // namespace fbfft_amd
