// The reference's two-call forms of the 64 x 64 and 128 x 128 transforms, kept
// for callers that already own the scratch buffer and issue both calls
// (forward: fbfft/FBFFT2D-inl.cuh:230-317 then :321-444; inverse:
// fbfft/FBIFFT2D-inl.cuh:252-356 then :360-474).  New code should use the
// single-kernel path in fft2d_large.hip, which produces the same result with one
// pass over HBM.
//
// All four passes are batches of N-point complex FFTs that differ only in how a
// transform's points are gathered and where its results go, so one kernel serves
// them: a 256-lane workgroup stages 256/G transforms in LDS (G = N/32 lanes per
// transform), runs the radix-G split + 32-point in-register FFT and scatters.
// The transposed reads of the second passes are coalesced by running the lanes
// along the transform index (consecutive transforms are adjacent in memory).
#include "common.h"
#include "fft_lds.h"
#include "fft_regs.h"

namespace fbfft_amd {
namespace {

constexpr int kTP = 256;

struct TwoPassArgs {
  float* src;      // real plane or complex-as-float
  float* dst;
  long s0, s1, s2;  // src strides (floats) of its three leading dims
  long d0, d1, d2;  // dst strides (floats)
  int B;            // planes (for the inverse: of the real / half-spectrum tensor)
  int h, w, padL, padU;
};

// MODE 0: forward pass 1   real [B][h][w] window      -> scratch [B][N][N/2+1]   (rows)
// MODE 1: forward pass 2   scratch [B][N][N/2+1]      -> dst [B][N/2+1][N]       (columns, transposed)
// MODE 2: inverse pass 1   src [B][N/2+1][N]          -> scratch [ceil(B/2)][N][N], planes paired
// MODE 3: inverse pass 2   scratch [ceil(B/2)][N][N]  -> real [B][h][w] window
template <int N, int MODE>
__global__ __launch_bounds__(kTP) void twoPassKernel(TwoPassArgs a, int total) {
  constexpr int G = N / 32, L = 32, ROWS = kTP / G, RS = N + 1, nc = N / 2 + 1;
  constexpr bool FWD = MODE < 2;
  __shared__ __align__(8) c32 lds[ROWS * RS];
  __shared__ __align__(8) c32 tw[256];
  const int t = threadIdx.x;
  const int q0 = blockIdx.x * ROWS;
  const int half = (a.B + 1) / 2;
  fillTwiddles<FWD>(tw, t, kTP);

  auto cplxAt = [](const float* p) { return *reinterpret_cast<const float2*>(p); };
  // Hermitian expansion of the half spectrum [N/2+1][N] (fbfft/FBIFFT2D-inl.cuh:61-97)
  // (one load at a selected address, so that the loads of a batch stay free of branches)
  auto expand = [&](int b, int row, int col) {
    const bool stored = row < nc;
    const int r = stored ? row : N - row, c = stored ? col : (N - col) % N;
    c32 v = cplxAt(a.src + (long)b * a.s0 + (long)r * a.s1 + (long)c * a.s2);
    return c32{v.x, stored ? v.y : -v.y};
  };

  // Gather ROWS transforms of N points.  Lanes run along whichever index is
  // contiguous in the source: the point index j for modes 0 and 2, the transform
  // index for modes 1 and 3 (the transposed reads of the second passes).  Loads go
  // out in batches of 16 at clamped coordinates with no branch between them; what
  // lies outside the window or beyond the last transform is zeroed or ignored later.
  constexpr bool ALONG_Q = MODE == 1 || MODE == 3;
  constexpr int ITER = ROWS * N / kTP, BATCH = 16;
  static_assert(ITER % BATCH == 0, "whole batches");
  // real rows on 16-byte boundaries, window edge and width multiples of 4: 16-byte loads
  const bool vec = MODE == 0 && a.s2 == 1 && ((a.s1 | a.s0 | a.padL | a.w) & 3) == 0 &&
                   (reinterpret_cast<uintptr_t>(a.src) & 15) == 0;
  if (vec) {
    constexpr int I4 = ITER / 4;  // 8 float4 per lane
    float v4[4 * I4];
#pragma unroll
    for (int u = 0; u < I4; ++u) {
      const int idx = t + kTP * u;
      const int qi = idx / (N / 4), j4 = idx % (N / 4);
      const int q = min(q0 + qi, total - 1);
      const int b = q / N, y = q % N;
      const int ys = min(max(y - a.padU, 0), a.h - 1), xs = min(max(4 * j4 - a.padL, 0), a.w - 4);
      const float4 w = *reinterpret_cast<const float4*>(a.src + (long)b * a.s0 + (long)ys * a.s1 + xs);
      v4[4 * u] = w.x;
      v4[4 * u + 1] = w.y;
      v4[4 * u + 2] = w.z;
      v4[4 * u + 3] = w.w;
    }
#pragma unroll
    for (int u = 0; u < I4; ++u) {
      const int idx = t + kTP * u;
      const int qi = idx / (N / 4), j4 = idx % (N / 4);
      const int y = min(q0 + qi, total - 1) % N;
      const bool in = inWindow(y, 4 * j4, a.padU, a.padL, a.h, a.w);
      c32* d = lds + qi * RS + 4 * j4;
#pragma unroll
      for (int e = 0; e < 4; ++e) d[e] = c32{in ? v4[4 * u + e] : 0.0f, 0.0f};
    }
  } else
#pragma unroll
  for (int i0 = 0; i0 < ITER; i0 += BATCH) {
    float vx[BATCH], vy[BATCH];
#pragma unroll
    for (int u = 0; u < BATCH; ++u) {
      const int idx = t + kTP * (i0 + u);
      const int qi = ALONG_Q ? idx % ROWS : idx / N, j = ALONG_Q ? idx / ROWS : idx % N;
      const int q = min(q0 + qi, total - 1);
      c32 v = c32{0.f, 0.f};
      if (MODE == 0) {
        const int b = q / N, y = q % N;
        const int ys = min(max(y - a.padU, 0), a.h - 1), xs = min(max(j - a.padL, 0), a.w - 1);
        v.x = a.src[(long)b * a.s0 + (long)ys * a.s1 + (long)xs * a.s2];
      } else if (MODE == 1) {
        const int b = q / nc, kx = q % nc;
        v = cplxAt(a.src + (long)b * a.s0 + (long)j * a.s1 + (long)kx * a.s2);
      } else if (MODE == 2) {
        const int b = q / N, row = q % N;
        v = expand(b, row, j);
        const c32 w = expand(min(b + half, a.B - 1), row, j);
        if (b + half < a.B) {
          v.x -= w.y;  // + i * w
          v.y += w.x;
        }
      } else {
        const int b = q / N, x = q % N;
        v = cplxAt(a.src + (long)b * a.s0 + (long)j * a.s1 + (long)x * a.s2);
      }
      vx[u] = v.x;
      vy[u] = v.y;
    }
#pragma unroll
    for (int u = 0; u < BATCH; ++u) {
      const int idx = t + kTP * (i0 + u);
      const int qi = ALONG_Q ? idx % ROWS : idx / N, j = ALONG_Q ? idx / ROWS : idx % N;
      c32 v = c32{vx[u], vy[u]};
      if (MODE == 0) {
        const int y = min(q0 + qi, total - 1) % N;
        if (!inWindow(y, j, a.padU, a.padL, a.h, a.w)) v.x = 0.0f;
      }
      lds[qi * RS + j] = v;
    }
  }
  __syncthreads();

  const int row = t % ROWS, g = t / ROWS;
  c32* z = lds + row * RS;
  c32 v[L];
  splitFFT<N, G, FWD>(z, g, tw, v);
  __syncthreads();
  staticFor<L>([&](auto kk) {
    constexpr int k = decltype(kk)::value;
    z[G * k + g] = v[slot<L>(k)];
  });
  __syncthreads();

  // results leave along their contiguous index k; the first forward pass keeps
  // N/2+1 of its N bins
  constexpr int KEEP = MODE == 0 ? nc : N;
#pragma unroll 4
  for (int idx = t; idx < ROWS * KEEP; idx += kTP) {
    const int qi = idx / KEEP, k = idx % KEEP;
    const int q = q0 + qi;
    if (q >= total) break;
    const c32 r = lds[qi * RS + k];
    if (MODE == 0) {
      const int b = q / N, y = q % N;
      *reinterpret_cast<float2*>(a.dst + (long)b * a.d0 + (long)y * a.d1 + (long)k * a.d2) = r;
    } else if (MODE == 1) {
      const int b = q / nc, kx = q % nc;
      *reinterpret_cast<float2*>(a.dst + (long)b * a.d0 + (long)kx * a.d1 + (long)k * a.d2) = r;
    } else if (MODE == 2) {
      const int b = q / N, rw = q % N;
      *reinterpret_cast<float2*>(a.dst + (long)b * a.d0 + (long)rw * a.d1 + (long)k * a.d2) = r;
    } else {
      const int b = q / N, x = q % N;  // x: output row, k: output column
      if (inWindow(x, k, a.padU, a.padL, a.h, a.w)) {
        const long o = (long)(x - a.padU) * a.d1 + (long)(k - a.padL) * a.d2;
        a.dst[(long)b * a.d0 + o] = r.x;
        if (b + half < a.B) a.dst[(long)(b + half) * a.d0 + o] = r.y;
      }
    }
  }
}

template <int N, int MODE>
int launchMode(const TwoPassArgs& a, hipStream_t s) {
  constexpr int ROWS = kTP / (N / 32), nc = N / 2 + 1;
  const int half = (a.B + 1) / 2;
  const int total = MODE == 0 ? a.B * N : MODE == 1 ? a.B * nc : half * N;
  if (total <= 0) return FBFFT_SUCCESS;
  twoPassKernel<N, MODE><<<dim3(ceilDiv(total, ROWS)), dim3(kTP), 0, s>>>(a, total);
  return launchStatus();
}

}  // namespace

int launchTwoPass(int N, int mode, float* src, long s0, long s1, long s2, float* dst, long d0,
                  long d1, long d2, int B, int h, int w, int padL, int padU, hipStream_t s) {
  TwoPassArgs a{src, dst, s0, s1, s2, d0, d1, d2, B, h, w, padL, padU};
  if (N == 64) {
    switch (mode) {
      case 0: return launchMode<64, 0>(a, s);
      case 1: return launchMode<64, 1>(a, s);
      case 2: return launchMode<64, 2>(a, s);
      case 3: return launchMode<64, 3>(a, s);
    }
  } else if (N == 128) {
    switch (mode) {
      case 0: return launchMode<128, 0>(a, s);
      case 1: return launchMode<128, 1>(a, s);
      case 2: return launchMode<128, 2>(a, s);
      case 3: return launchMode<128, 3>(a, s);
    }
  }
  return FBFFT_UNSUPPORTED_SIZE;
}

}  // namespace fbfft_amd
