// FFT building blocks that read their input from LDS: the radix-G
// decimation-in-frequency split that lets G lanes share one long transform, and
// the full-circle twiddle table they index at run time.
#pragma once

#include "fft_regs.h"

namespace fbfft_amd {

// tw[m] = e^{-/+ 2 pi i m / 256}, m = 0..255 (forward: minus), expanded from the
// half-circle table; every entry is an exact table value or its negation.
template <bool FWD>
__device__ __forceinline__ void fillTwiddles(c32* tw, int t, int threads) {
  for (int m = t; m < 256; m += threads) {
    const int h = m & 127;
    float c = __builtin_bit_cast(float, kTwiddleBits[2 * h]);
    float s = __builtin_bit_cast(float, kTwiddleBits[2 * h + 1]);
    if (m >= 128) {
      c = -c;
      s = -s;
    }
    tw[m] = c32{c, FWD ? -s : s};
  }
}

// Lane g of G computes outputs X[G*k + g], k = 0..N/G-1, of the N-point FFT of
// col[0..N) (LDS, unit stride); they are left in v[slot<N/G>(k)].  G = 1 is the
// plain in-register transform.
template <int N, int G, bool FWD>
__device__ __forceinline__ void splitFFT(const c32* col, int g, const c32* tw, c32 (&v)[N / G]) {
  constexpr int L = N / G;
  static_assert(G == 1 || G == 2 || G == 4, "split factor");
  if constexpr (G == 1) {
    staticFor<L>([&](auto jj) {
      constexpr int j = decltype(jj)::value;
      v[j] = col[j];
    });
  } else if constexpr (G == 2) {
    const float sgn = g ? -1.0f : 1.0f;
    staticFor<L>([&](auto jj) {
      constexpr int j = decltype(jj)::value;
      c32 u0 = col[j], u1 = col[j + L];
      c32 comb = c32{u0.x + sgn * u1.x, u0.y + sgn * u1.y};
      c32 w = tw[(g * (j * (256 / N))) & 255];
      v[j] = cmul(comb, w);
    });
  } else {
    const float sA = (g & 1) ? -1.0f : 1.0f;
    const bool rot = (g & 1) != 0;
    // forward: omega = -i  -> g=1: -i*b, g=3: +i*b;  inverse: the other way round
    const float sB = (g == 0) ? 1.0f : (g == 2) ? -1.0f : ((g == 1) == FWD) ? -1.0f : 1.0f;
    staticFor<L>([&](auto jj) {
      constexpr int j = decltype(jj)::value;
      c32 u0 = col[j], u1 = col[j + L], u2 = col[j + 2 * L], u3 = col[j + 3 * L];
      c32 a = c32{u0.x + sA * u2.x, u0.y + sA * u2.y};
      c32 b = c32{u1.x + sA * u3.x, u1.y + sA * u3.y};
      c32 br = rot ? c32{-b.y, b.x} : b;  // i*b when rot
      c32 comb = c32{a.x + sB * br.x, a.y + sB * br.y};
      c32 w = tw[(g * (j * (256 / N))) & 255];
      v[j] = cmul(comb, w);
    });
  }
  regFFT<L, FWD>(v);
}

}  // namespace fbfft_amd
