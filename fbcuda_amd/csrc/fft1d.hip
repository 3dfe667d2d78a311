// Batched 1D real-to-complex / complex-to-real transforms, N = 2 .. 256
// (replaces decimateInFrequency1DKernel, fbfft/FBFFTCommon.cuh:710-833, and its
// dispatch tables in fbfft/FBFFT-inl.cuh:19-150).
//
// A workgroup of 256 lanes stages ROWS = 256/G rows in LDS with coalesced
// 8-byte accesses.  Each row is transformed as an N/2-point complex FFT of the
// even/odd packing z[j] = x[2j] + i x[2j+1]: one lane per row up to N = 64, two
// lanes for N = 128 and four for N = 256 (radix-G split read straight from LDS,
// 32 points per lane in VGPRs, G uniform per wave).  The real-input fix-up runs
// on the way out (forward) or on the way in (inverse) with lanes mapped to
// consecutive output elements, so HBM stores are contiguous.  The reference
// instead pairs two rows into one N-point complex transform; results agree to
// rounding and rows never depend on their neighbours here, so odd batch sizes
// need no special case.
#include "common.h"
#include "fft_lds.h"
#include "fft_regs.h"

namespace fbfft_amd {
namespace {

constexpr int k1dThreads = 256;

template <int N>
struct Cfg1D {
  static constexpr int H = N / 2;
  static constexpr int G = (H <= 32) ? 1 : H / 32;
  static constexpr int L = H / G;
  static constexpr int ROWS = k1dThreads / G;
  static constexpr int RS = H + 1;  // LDS row stride in complex (= N + 2 floats)
};

// real [B][N] with strides (sb, sx); cplx [B][N/2+1][2] with strides (cb, ck)
struct Row1D {
  float* real;
  int sb, sx;
  float* cplx;
  int cb, ck;
  int B;
  int padL;
};

template <int N, bool FAST>
__global__ __launch_bounds__(k1dThreads) void fft1dForward(Row1D a) {
  using C = Cfg1D<N>;
  constexpr int H = C::H, G = C::G, L = C::L, ROWS = C::ROWS, RS = C::RS;
  __shared__ __align__(16) c32 lds[ROWS * RS];
  __shared__ __align__(8) c32 tw[256];
  const int t = threadIdx.x;
  const int b0 = blockIdx.x * ROWS;
  fillTwiddles<true>(tw, t, k1dThreads);

  // ---- rows -> LDS as packed complex z[j] = (x[2j], x[2j+1]); every load is
  // issued before the first one is consumed ----
  constexpr int LOADS = (ROWS * H + k1dThreads - 1) / k1dThreads;
  c32 in[LOADS];
  staticFor<LOADS>([&](auto ii) {
    constexpr int i = decltype(ii)::value;
    const int idx = t + k1dThreads * i;
    const int row = min(idx / H, ROWS - 1), j = idx % H;
    const int b = min(b0 + row, a.B - 1);
    if constexpr (FAST) {
      in[i] = *reinterpret_cast<const float2*>(a.real + (size_t)b * a.sb + 2 * j);
    } else {
      const float* src = a.real + (size_t)b * a.sb;
      const int x0 = 2 * j - a.padL, x1 = 2 * j + 1 - a.padL;
      // a right shift that drops the last padL samples (fbfft/FBFFTCommon.cuh:325)
      in[i].x = x0 >= 0 ? src[(size_t)x0 * a.sx] : 0.0f;
      in[i].y = x1 >= 0 ? src[(size_t)x1 * a.sx] : 0.0f;
    }
  });
  staticFor<LOADS>([&](auto ii) {
    constexpr int i = decltype(ii)::value;
    const int idx = t + k1dThreads * i;
    if (idx < ROWS * H) lds[(idx / H) * RS + idx % H] = in[i];
  });
  __syncthreads();

  const int row = t % ROWS, g = t / ROWS;
  c32* zrow = lds + row * RS;
  c32 v[L];
  splitFFT<H, G, true>(zrow, g, tw, v);
  __syncthreads();
  staticFor<L>([&](auto kk) {
    constexpr int k = decltype(kk)::value;
    zrow[G * k + g] = v[slot<L>(k)];
  });
  __syncthreads();

  // ---- fix-up and store: lanes run over consecutive output bins ----
  for (int idx = t; idx < ROWS * (H + 1); idx += k1dThreads) {
    const int r = idx / (H + 1), k = idx % (H + 1);
    const int b = b0 + r;
    if (b >= a.B) break;
    const c32* z = lds + r * RS;
    c32 f;
    if (k == 0 || k == H) {
      c32 z0 = z[0];
      f = c32{k == 0 ? z0.x + z0.y : z0.x - z0.y, 0.0f};
    } else {
      c32 p = z[k], q = z[H - k];
      c32 e = c32{0.5f * (p.x + q.x), 0.5f * (p.y - q.y)};
      c32 o = c32{0.5f * (p.y + q.y), -0.5f * (p.x - q.x)};
      c32 w = tw[k * (256 / N)];
      c32 wo = cmul(o, w);
      f = c32{e.x + wo.x, e.y + wo.y};
    }
    *reinterpret_cast<float2*>(a.cplx + (size_t)b * a.cb + (size_t)k * a.ck) = f;
  }
}

template <int N, bool FAST>
__global__ __launch_bounds__(k1dThreads) void fft1dInverse(Row1D a) {
  using C = Cfg1D<N>;
  constexpr int H = C::H, G = C::G, L = C::L, ROWS = C::ROWS, RS = C::RS;
  __shared__ __align__(16) c32 lds[ROWS * RS];
  __shared__ __align__(8) c32 tw[256];
  const int t = threadIdx.x;
  const int b0 = blockIdx.x * ROWS;
  fillTwiddles<false>(tw, t, k1dThreads);

  // ---- spectra -> LDS, all loads in flight together ----
  constexpr int LOADS = (ROWS * (H + 1) + k1dThreads - 1) / k1dThreads;
  c32 in[LOADS];
  staticFor<LOADS>([&](auto ii) {
    constexpr int i = decltype(ii)::value;
    const int idx = t + k1dThreads * i;
    const int r = min(idx / (H + 1), ROWS - 1), k = idx % (H + 1);
    const int b = min(b0 + r, a.B - 1);
    in[i] = *reinterpret_cast<const float2*>(a.cplx + (size_t)b * a.cb + (size_t)k * a.ck);
  });
  staticFor<LOADS>([&](auto ii) {
    constexpr int i = decltype(ii)::value;
    const int idx = t + k1dThreads * i;
    if (idx < ROWS * (H + 1)) lds[(idx / (H + 1)) * RS + idx % (H + 1)] = in[i];
  });
  __syncthreads();

  // ---- inverse real fix-up in place: bins k and H-k form one work item ----
  for (int idx = t; idx < ROWS * (H / 2 + 1); idx += k1dThreads) {
    const int r = idx / (H / 2 + 1), k = idx % (H / 2 + 1);
    c32* z = lds + r * RS;
    if (k == 0) {
      // only the real parts of F[0] and F[N/2] reach a real result
      const float f0 = z[0].x, fh = z[H].x;
      z[0] = c32{f0 + fh, f0 - fh};
    } else if (2 * k == H) {
      c32 p = z[k];
      z[k] = c32{2.0f * p.x, -2.0f * p.y};
    } else {
      c32 p = z[k], q = z[H - k];
      c32 e = c32{p.x + q.x, p.y - q.y};
      c32 d = c32{p.x - q.x, p.y + q.y};
      c32 o = cmul(d, tw[k * (256 / N)]);
      z[k] = c32{e.x - o.y, e.y + o.x};
      z[H - k] = c32{e.x + o.y, o.x - e.y};
    }
  }
  __syncthreads();

  const int row = t % ROWS, g = t / ROWS;
  c32* zrow = lds + row * RS;
  c32 v[L];
  splitFFT<H, G, false>(zrow, g, tw, v);
  __syncthreads();
  staticFor<L>([&](auto kk) {
    constexpr int k = decltype(kk)::value;
    zrow[G * k + g] = v[slot<L>(k)];
  });
  __syncthreads();

  // ---- store rows ----
  for (int idx = t; idx < ROWS * H; idx += k1dThreads) {
    const int r = idx / H, j = idx % H;
    const int b = b0 + r;
    if (b >= a.B) break;
    c32 val = lds[r * RS + j];
    if constexpr (FAST) {
      *reinterpret_cast<float2*>(a.real + (size_t)b * a.sb + 2 * j) = val;
    } else {
      // the reference writes the first row of each pair at x and the second at
      // x - padL, both only for x >= padL (fbfft/FBFFTCommon.cuh:423-428)
      float* dst = a.real + (size_t)b * a.sb;
      const int shift = (b & 1) ? a.padL : 0;
      const int x0 = 2 * j, x1 = 2 * j + 1;
      if (x0 >= a.padL) dst[(size_t)(x0 - shift) * a.sx] = val.x;
      if (x1 >= a.padL) dst[(size_t)(x1 - shift) * a.sx] = val.y;
    }
  }
}

template <int N>
int launch1d(bool forward, const Row1D& a, bool fast, hipStream_t s) {
  dim3 grid(ceilDiv(a.B, Cfg1D<N>::ROWS)), block(k1dThreads);
  if (forward) {
    if (fast)
      fft1dForward<N, true><<<grid, block, 0, s>>>(a);
    else
      fft1dForward<N, false><<<grid, block, 0, s>>>(a);
  } else {
    if (fast)
      fft1dInverse<N, true><<<grid, block, 0, s>>>(a);
    else
      fft1dInverse<N, false><<<grid, block, 0, s>>>(a);
  }
  return launchStatus();
}

}  // namespace

int launchFft1d(bool forward, int N, float* real, int sb, int sx, float* cplx, int cb, int ck,
                int B, int padL, hipStream_t s) {
  if (B <= 0) return FBFFT_SUCCESS;
  Row1D a{real, sb, sx, cplx, cb, ck, B, padL};
  const bool fast = padL == 0 && sx == 1 && sb % 2 == 0 && aligned(real, 8);
  switch (N) {
    case 2: return launch1d<2>(forward, a, fast, s);
    case 4: return launch1d<4>(forward, a, fast, s);
    case 8: return launch1d<8>(forward, a, fast, s);
    case 16: return launch1d<16>(forward, a, fast, s);
    case 32: return launch1d<32>(forward, a, fast, s);
    case 64: return launch1d<64>(forward, a, fast, s);
    case 128: return launch1d<128>(forward, a, fast, s);
    case 256: return launch1d<256>(forward, a, fast, s);
  }
  return FBFFT_UNSUPPORTED_SIZE;
}

}  // namespace fbfft_amd
