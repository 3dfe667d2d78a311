// In-register FFT building blocks for gfx950.
//
// Every transform here runs inside one lane on a small array of complex values
// that the compiler keeps in VGPRs: all indices and all twiddle factors are
// compile-time constants, so a butterfly is a handful of v_add/v_sub/v_fma with
// literal operands and no cross-lane traffic.  The twiddles come from the same
// correctly-rounded 128-entry table the reference uses (fbfft/Twiddles.cuh:322-453).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>
#include <utility>

namespace fbfft_amd {

typedef float2 c32;

constexpr uint32_t kTwiddleBits[256] = {
#include "twiddles_f32.inc"
};

// e^{+i*pi*IDX/128}
template <int IDX>
struct TableEntry {
  static_assert(IDX >= 0 && IDX < 128, "twiddle index out of range");
  static constexpr float c = __builtin_bit_cast(float, kTwiddleBits[2 * IDX]);
  static constexpr float s = __builtin_bit_cast(float, kTwiddleBits[2 * IDX + 1]);
};

// compile-time loop: f(std::integral_constant<int, 0>{}) ... f(<N-1>)
template <typename F, int... Is>
__device__ __forceinline__ void staticForImpl(F&& f, std::integer_sequence<int, Is...>) {
  (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void staticFor(F&& f) {
  staticForImpl(static_cast<F&&>(f), std::make_integer_sequence<int, N>{});
}

constexpr int ilog2(int n) { return n <= 1 ? 0 : 1 + ilog2(n / 2); }

constexpr int bitrev(int x, int bits) {
  int r = 0;
  for (int i = 0; i < bits; ++i) r |= ((x >> i) & 1) << (bits - 1 - i);
  return r;
}

__device__ __forceinline__ c32 cadd(c32 a, c32 b) { return c32{a.x + b.x, a.y + b.y}; }
__device__ __forceinline__ c32 csub(c32 a, c32 b) { return c32{a.x - b.x, a.y - b.y}; }
__device__ __forceinline__ c32 cmul(c32 a, c32 b) {
  return c32{a.x * b.x - a.y * b.y, a.x * b.y + a.y * b.x};
}
__device__ __forceinline__ c32 cconj(c32 a) { return c32{a.x, -a.y}; }

// d * W, W = e^{-/+ 2*pi*i*K/M} (forward: minus), K in [0, M/2)
template <int M, int K, bool FWD>
__device__ __forceinline__ c32 mulRoot(c32 d) {
  static_assert(K >= 0 && 2 * K < M, "root index");
  if constexpr (K == 0) {
    return d;
  } else if constexpr (4 * K == M) {
    return FWD ? c32{d.y, -d.x} : c32{-d.y, d.x};
  } else if constexpr (8 * K == M) {
    constexpr float h = TableEntry<32>::c;  // sqrt(1/2)
    return FWD ? c32{(d.x + d.y) * h, (d.y - d.x) * h} : c32{(d.x - d.y) * h, (d.x + d.y) * h};
  } else if constexpr (8 * K == 3 * M) {
    constexpr float h = TableEntry<32>::c;
    return FWD ? c32{(d.y - d.x) * h, -(d.x + d.y) * h} : c32{-(d.x + d.y) * h, (d.x - d.y) * h};
  } else {
    constexpr float c = TableEntry<K * 256 / M>::c;
    constexpr float s = FWD ? -TableEntry<K * 256 / M>::s : TableEntry<K * 256 / M>::s;
    return c32{d.x * c - d.y * s, d.x * s + d.y * c};
  }
}

// d * W / 2 with the same W: the halving is folded into the literals
template <int M, int K, bool FWD>
__device__ __forceinline__ c32 mulHalfRoot(c32 d) {
  static_assert(K >= 0 && 2 * K < M, "root index");
  if constexpr (K == 0) {
    return c32{0.5f * d.x, 0.5f * d.y};
  } else if constexpr (4 * K == M) {
    return FWD ? c32{0.5f * d.y, -0.5f * d.x} : c32{-0.5f * d.y, 0.5f * d.x};
  } else if constexpr (8 * K == M) {
    constexpr float h = 0.5f * TableEntry<32>::c;
    return FWD ? c32{(d.x + d.y) * h, (d.y - d.x) * h} : c32{(d.x - d.y) * h, (d.x + d.y) * h};
  } else if constexpr (8 * K == 3 * M) {
    constexpr float h = 0.5f * TableEntry<32>::c;
    return FWD ? c32{(d.y - d.x) * h, -(d.x + d.y) * h} : c32{-(d.x + d.y) * h, (d.x - d.y) * h};
  } else {
    constexpr float c = 0.5f * TableEntry<K * 256 / M>::c;
    constexpr float s = 0.5f * (FWD ? -TableEntry<K * 256 / M>::s : TableEntry<K * 256 / M>::s);
    return c32{d.x * c - d.y * s, d.x * s + d.y * c};
  }
}

// One decimation-in-time butterfly with the twiddle folded into the additions:
// (a, b) <- (a + W b, a - W b), W = e^{-/+ 2*pi*i*K/M} (forward: minus), K in [0, M/2).
// A general W = c + i s costs six multiply-adds instead of the eight instructions of
// "multiply, then add and subtract": with t = s / c, W b = c (b.x - t b.y, b.y + t b.x),
// so two multiply-adds form the bracket and four more apply c while adding to a (the
// bracket is taken relative to the larger of |c| and |s|, so |t| <= 1).  The roots on the
// diagonals cost two additions and four multiply-adds, +-1 and +-i four additions.
template <int M, int K, bool FWD>
__device__ __forceinline__ void butterfly(c32& a, c32& b) {
  static_assert(K >= 0 && 2 * K < M, "root index");
  const c32 p = a, q = b;
  if constexpr (K == 0) {
    a = cadd(p, q);
    b = csub(p, q);
  } else if constexpr (4 * K == M) {  // W = -i (forward), +i (inverse)
    if constexpr (FWD) {
      a = c32{p.x + q.y, p.y - q.x};
      b = c32{p.x - q.y, p.y + q.x};
    } else {
      a = c32{p.x - q.y, p.y + q.x};
      b = c32{p.x + q.y, p.y - q.x};
    }
  } else if constexpr (8 * K == M || 8 * K == 3 * M) {
    constexpr float h = TableEntry<32>::c;  // sqrt(1/2)
    // W q = h (u, v)
    float u, v;
    if constexpr (8 * K == M) {
      u = FWD ? q.x + q.y : q.x - q.y;
      v = FWD ? q.y - q.x : q.x + q.y;
    } else {
      u = FWD ? q.y - q.x : -(q.x + q.y);
      v = FWD ? -(q.x + q.y) : q.x - q.y;
    }
    a = c32{__builtin_fmaf(h, u, p.x), __builtin_fmaf(h, v, p.y)};
    b = c32{__builtin_fmaf(-h, u, p.x), __builtin_fmaf(-h, v, p.y)};
  } else {
    constexpr float c = TableEntry<K * 256 / M>::c;
    constexpr float s = FWD ? -TableEntry<K * 256 / M>::s : TableEntry<K * 256 / M>::s;
    constexpr bool byCos = (c < 0 ? -c : c) >= (s < 0 ? -s : s);
    if constexpr (byCos) {
      constexpr float t = (float)((double)s / (double)c);
      const float u = __builtin_fmaf(-t, q.y, q.x), v = __builtin_fmaf(t, q.x, q.y);
      a = c32{__builtin_fmaf(c, u, p.x), __builtin_fmaf(c, v, p.y)};
      b = c32{__builtin_fmaf(-c, u, p.x), __builtin_fmaf(-c, v, p.y)};
    } else {
      // W q = s (t q.x - q.y, q.x + t q.y), t = c / s
      constexpr float t = (float)((double)c / (double)s);
      const float u = __builtin_fmaf(t, q.x, -q.y), v = __builtin_fmaf(t, q.y, q.x);
      a = c32{__builtin_fmaf(s, u, p.x), __builtin_fmaf(s, v, p.y)};
      b = c32{__builtin_fmaf(-s, u, p.x), __builtin_fmaf(-s, v, p.y)};
    }
  }
}

// In-register FFT of a[0..N): natural order in, bit-reversed order out (the value with
// frequency index k ends up in a[bitrev(k)] = a[slot<N>(k)]).  Radix-2 decimation in
// time run on renamed registers: logical position i of the textbook algorithm
// (bit-reversed input, natural output) is register a[bitrev(i)], so the caller's
// natural-order input is already in place and the output lands where a decimation in
// frequency would have left it.  32 points: 388 vector instructions where the
// decimation-in-frequency form (add, subtract, then multiply) took 456.
template <int N, bool FWD, int M = 2>
__device__ __forceinline__ void regFFT(c32 (&a)[N]) {
  if constexpr (M <= N) {
    constexpr int half = M / 2;
    constexpr int bits = ilog2(N);
    staticFor<N / M>([&](auto blk) {
      staticFor<half>([&](auto kk) {
        constexpr int k = decltype(kk)::value;
        constexpr int lo = bitrev(decltype(blk)::value * M + k, bits);
        constexpr int hi = bitrev(decltype(blk)::value * M + k + half, bits);
        butterfly<M, k, FWD>(a[lo], a[hi]);
      });
    });
    regFFT<N, FWD, 2 * M>(a);
  }
}

// index of frequency k in the output of regFFT<N>
template <int N>
constexpr int slot(int k) {
  return bitrev(k, ilog2(N));
}

// F[K] and F[H-K] of the N = 2H-point real transform from a = Z[K], b = Z[H-K] of
// the H-point transform of the even/odd packing:
// E = (a + conj b)/2, O = -i (a - conj b)/2, T = W_N^K O, F[K] = E + T,
// F[H-K] = conj(E - T).  The halvings ride on the twiddle's literals and on the
// final multiply-adds: 12 instructions per pair, not 16.
template <int N, int K>
__device__ __forceinline__ void realPairForward(c32 a, c32 b, c32& fk, c32& fhk) {
  const c32 e2 = c32{a.x + b.x, a.y - b.y};
  const c32 o2 = c32{a.y + b.y, b.x - a.x};
  const c32 t = mulHalfRoot<N, K, true>(o2);
  fk = c32{__builtin_fmaf(0.5f, e2.x, t.x), __builtin_fmaf(0.5f, e2.y, t.y)};
  fhk = c32{__builtin_fmaf(0.5f, e2.x, -t.x), __builtin_fmaf(-0.5f, e2.y, t.y)};
}

// Forward real-input fix-up.  z (in regFFT output order) is the H-point complex
// FFT of z[j] = x[2j] + i*x[2j+1].  emit(k, value) is called once for every
// k = 0..H-1 (k as an integral_constant) with F[k] of the 2H-point real
// transform; for k = 0 the value is (F[0], F[H]) packed as (re, im) - both are
// real.  Bins k and H-k share one twiddle product.
template <int H, typename Emit>
__device__ __forceinline__ void realFixupForwardEmit(const c32 (&z)[H], Emit&& emit) {
  constexpr int N = 2 * H;
  {
    c32 z0 = z[0];
    emit(std::integral_constant<int, 0>{}, c32{z0.x + z0.y, z0.x - z0.y});
  }
  staticFor<H / 2 - 1>([&](auto kk) {
    constexpr int k = decltype(kk)::value + 1;
    c32 a = z[slot<H>(k)];
    c32 b = z[slot<H>(H - k)];
    c32 fk, fhk;
    realPairForward<N, k>(a, b, fk, fhk);
    emit(std::integral_constant<int, k>{}, fk);
    emit(std::integral_constant<int, H - k>{}, fhk);
  });
  if constexpr (H >= 2) {
    c32 a = z[slot<H>(H / 2)];
    emit(std::integral_constant<int, H / 2>{}, c32{a.x, -a.y});
  }
}

template <int H>
__device__ __forceinline__ void realFixupForward(const c32 (&z)[H], c32 (&p)[H]) {
  realFixupForwardEmit<H>(z, [&](auto kk, c32 v) { p[decltype(kk)::value] = v; });
}

// Inverse of the above without the 1/2 factors (gain 2).  fetch(k) returns F[k]
// for k = 0..H-1 (k = 0: the packed (F[0], F[H])); z receives, in NATURAL order,
// the input of an inverse H-point complex FFT whose output is
// z[j] = (x[2j], x[2j+1]) * gain.
template <int H, typename Fetch>
__device__ __forceinline__ void realFixupInverseFetch(Fetch&& fetch, c32 (&z)[H]) {
  constexpr int N = 2 * H;
  {
    c32 p0 = fetch(std::integral_constant<int, 0>{});
    z[0] = c32{p0.x + p0.y, p0.x - p0.y};
  }
  staticFor<H / 2 - 1>([&](auto kk) {
    constexpr int k = decltype(kk)::value + 1;
    c32 a = fetch(std::integral_constant<int, k>{});
    c32 b = fetch(std::integral_constant<int, H - k>{});
    // E2 = a + conj b, O2 = (a - conj b) W_N^{-k}:
    // Z[k] = E2 + i O2, Z[H-k] = conj(E2) + i conj(O2)
    c32 e = c32{a.x + b.x, a.y - b.y};
    c32 d = c32{a.x - b.x, a.y + b.y};
    c32 o = mulRoot<N, k, false>(d);
    z[k] = c32{e.x - o.y, e.y + o.x};
    z[H - k] = c32{e.x + o.y, o.x - e.y};
  });
  if constexpr (H >= 2) {
    c32 a = fetch(std::integral_constant<int, H / 2>{});
    z[H / 2] = c32{2.0f * a.x, -2.0f * a.y};
  }
}

template <int H>
__device__ __forceinline__ void realFixupInverse(const c32 (&p)[H], c32 (&z)[H]) {
  realFixupInverseFetch<H>([&](auto kk) { return p[decltype(kk)::value]; }, z);
}

}  // namespace fbfft_amd
