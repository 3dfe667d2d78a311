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

// ---- N = 8 ... 256 with contiguous, 16-byte aligned operands ----
//
// Same staging as above, but the real-input fix-up never makes a pass of its own
// through LDS: with one lane per row (N <= 64) the whole half-length transform is in
// the lane's registers, and with two lanes per row (N = 128) the split is chosen so
// that the fix-up pairs (k, N/2 - k) stay inside one lane - the forward transform
// splits its outputs by parity, the inverse its inputs (E = IFFT(z even),
// O = IFFT(z odd), x[j] = E[j] + w^j O[j], x[j + N/4] = E[j] - w^j O[j], summed on
// the way out of LDS).  With four lanes per row (N = 256) the classes k = 0 and
// 2 mod 4 still pair inside their lane; lanes 1 and 3 hold each other's partners:
// forward each parks half of its transform in the row and finishes the pairs of
// its other half, inverse each derives its own inputs from the pairs (the
// partner's half of a pair is computed and dropped).  Spectra and rows then move between LDS and
// HBM as plain 16-byte streams.
template <int N>
struct CfgMid {
  static_assert(N >= 8 && N <= 256, "one lane per row up to 64 points, then two or four");
  static constexpr int H = N / 2;
  static constexpr int G = N <= 64 ? 1 : N / 64;  // lanes per row
  static constexpr int Q = H / G;           // points per lane (32)
  static constexpr int ROWS = k1dThreads / G;
  static constexpr int RS = H + 1;          // LDS row stride (complex) = spectrum row length
};

template <int N>
__global__ __launch_bounds__(k1dThreads, 2) void fft1dMidForward(const float* __restrict__ real,
                                                              float* __restrict__ cplx, int B) {
  using C = CfgMid<N>;
  constexpr int H = C::H, G = C::G, Q = C::Q, ROWS = C::ROWS, RS = C::RS;
  __shared__ __align__(16) c32 lds[ROWS * RS];
  __shared__ __align__(8) c32 tw[256];
  const int t = threadIdx.x;
  const int b0 = blockIdx.x * ROWS;
  const int rows = min(ROWS, B - b0);
  if constexpr (G > 1) fillTwiddles<true>(tw, t, k1dThreads);

  // ---- rows -> LDS as packed complex z[j] = (x[2j], x[2j+1]), 16 bytes per load ----
  constexpr int LOADS = ROWS * H / 2 / k1dThreads;
  const float4* src = reinterpret_cast<const float4*>(real + (size_t)b0 * N);
  float4 in[LOADS];
  staticFor<LOADS>([&](auto ii) {
    constexpr int i = decltype(ii)::value;
    const int idx = t + k1dThreads * i;               // float4 index: row = idx / (H/2)
    in[i] = src[min(idx, rows * (H / 2) - 1)];
  });
  staticFor<LOADS>([&](auto ii) {
    constexpr int i = decltype(ii)::value;
    const int idx = t + k1dThreads * i;
    c32* d = lds + (idx / (H / 2)) * RS + 2 * (idx % (H / 2));
    d[0] = c32{in[i].x, in[i].y};
    d[1] = c32{in[i].z, in[i].w};
  });
  __syncthreads();

  // ROWS is a multiple of 64: g is the same for a whole wave, and says so
  const int row = t % ROWS, g = __builtin_amdgcn_readfirstlane(t / ROWS);
  c32* zrow = lds + row * RS;
  c32 v[Q];
  if constexpr (G == 1) {
    splitFFT<H, 1, true>(zrow, 0, tw, v);
    // the row is this lane's alone and is in registers: overwrite it with F[0..H]
    realFixupForwardEmit<H>(v, [&](auto kk, c32 val) {
      constexpr int k = decltype(kk)::value;
      if constexpr (k == 0) {
        zrow[0] = c32{val.x, 0.0f};
        zrow[H] = c32{val.y, 0.0f};
      } else {
        zrow[k] = val;
      }
    });
  } else if constexpr (G == 4) {
    splitFFT<H, 4, true>(zrow, g, tw, v);   // lane g: Z[4k + g]; g is the wave index
    // The results are consumed in per-wave branches below the barrier.  Without this
    // the compiler sinks the whole transform into those branches and keeps the 128
    // raw values it was computed from alive across the barrier instead of the 32 results.
#pragma unroll
    for (int j = 0; j < Q; ++j) asm volatile("" : "+v"(v[j].x), "+v"(v[j].y));
    __syncthreads();                        // all four lanes of a row have read it
    // F[k] and F[H-k] from a = Z[k], b = Z[H-k]
    auto fixBoth = [&](auto kp, c32 a, c32 bq) __attribute__((always_inline)) {
      constexpr int k = decltype(kp)::value;
      c32 fk, fhk;
      realPairForward<N, k>(a, bq, fk, fhk);
      zrow[k] = fk;
      zrow[H - k] = fhk;
    };
    if (g == 0) {
      const c32 z0 = v[0];
      zrow[0] = c32{z0.x + z0.y, 0.0f};
      zrow[H] = c32{z0.x - z0.y, 0.0f};
      staticFor<Q / 2 - 1>([&](auto kk) {
        constexpr int k = decltype(kk)::value + 1;  // bins 4k and H-4k
        fixBoth(std::integral_constant<int, 4 * k>{}, v[slot<Q>(k)], v[slot<Q>(Q - k)]);
      });
      const c32 m = v[slot<Q>(Q / 2)];  // bin H/2
      zrow[H / 2] = c32{m.x, -m.y};
    } else if (g == 2) {
      staticFor<Q / 2>([&](auto kk) {
        constexpr int k = decltype(kk)::value;  // bins 4k+2 and H-4k-2
        fixBoth(std::integral_constant<int, 4 * k + 2>{}, v[slot<Q>(k)], v[slot<Q>(Q - 1 - k)]);
      });
    } else {
      // lanes 1 and 3: bin 4k+g pairs with H-4k-g = 4(Q-1-k) + (4-g), the other lane's.
      // Each parks the upper half of its transform (k >= Q/2) at its natural positions ...
      staticFor<Q / 2>([&](auto kk) {
        constexpr int k = decltype(kk)::value + Q / 2;
        zrow[4 * k + g] = v[slot<Q>(k)];
      });
    }
    __syncthreads();
    // ... and finishes the pairs of its own lower half: it alone reads and then
    // overwrites the partner's parked values, and nobody reads its lower positions.
    if (g == 1) {
      staticFor<Q / 2>([&](auto kk) {
        constexpr int k = decltype(kk)::value;
        fixBoth(std::integral_constant<int, 4 * k + 1>{}, v[slot<Q>(k)], zrow[H - (4 * k + 1)]);
      });
    } else if (g == 3) {
      staticFor<Q / 2>([&](auto kk) {
        constexpr int k = decltype(kk)::value;
        fixBoth(std::integral_constant<int, 4 * k + 3>{}, v[slot<Q>(k)], zrow[H - (4 * k + 3)]);
      });
    }
  } else {
    splitFFT<H, 2, true>(zrow, g, tw, v);   // lane g: Z[2k + g]
    __syncthreads();                        // both lanes of a row have read it
    auto pairOut = [&](auto kp, c32 a, c32 bq) __attribute__((always_inline)) {
      constexpr int k = decltype(kp)::value;  // bin k pairs with H-k
      c32 fk, fhk;
      realPairForward<N, k>(a, bq, fk, fhk);
      zrow[k] = fk;
      zrow[H - k] = fhk;
    };
    if (g == 0) {
      const c32 z0 = v[0];
      zrow[0] = c32{z0.x + z0.y, 0.0f};
      zrow[H] = c32{z0.x - z0.y, 0.0f};
      staticFor<Q / 2 - 1>([&](auto kk) {
        constexpr int k = decltype(kk)::value + 1;  // bins 2k and H-2k
        pairOut(std::integral_constant<int, 2 * k>{}, v[slot<Q>(k)], v[slot<Q>(Q - k)]);
      });
      const c32 m = v[slot<Q>(Q / 2)];  // bin H/2
      zrow[H / 2] = c32{m.x, -m.y};
    } else {
      staticFor<Q / 2>([&](auto kk) {
        constexpr int k = decltype(kk)::value;  // bins 2k+1 and H-2k-1
        pairOut(std::integral_constant<int, 2 * k + 1>{}, v[slot<Q>(k)], v[slot<Q>(Q - 1 - k)]);
      });
    }
  }
  __syncthreads();

  // ---- spectra out: LDS and HBM hold the same [row][H+1] stream ----
  const int total = rows * RS;  // complex values of this workgroup
  float4* dst = reinterpret_cast<float4*>(cplx + (size_t)b0 * 2 * RS);
  const float4* l4 = reinterpret_cast<const float4*>(lds);
  for (int q = t; q < total / 2; q += k1dThreads) streamStore(dst + q, l4[q]);
  if ((total & 1) && t == 0)
    reinterpret_cast<float2*>(cplx + (size_t)b0 * 2 * RS)[total - 1] = lds[total - 1];
}

template <int N>
__global__ __launch_bounds__(k1dThreads, 2) void fft1dMidInverse(const float* __restrict__ cplx,
                                                              float* __restrict__ real, int B) {
  using C = CfgMid<N>;
  constexpr int H = C::H, G = C::G, Q = C::Q, ROWS = C::ROWS, RS = C::RS;
  __shared__ __align__(16) c32 lds[ROWS * RS];
  const int t = threadIdx.x;
  const int b0 = blockIdx.x * ROWS;
  const int rows = min(ROWS, B - b0);

  // ---- spectra -> LDS, the same [row][H+1] stream in both places ----
  const int total = rows * RS;
  constexpr int LOADS = (ROWS * RS / 2 + k1dThreads - 1) / k1dThreads;
  const float4* src = reinterpret_cast<const float4*>(cplx + (size_t)b0 * 2 * RS);
  float in[4 * LOADS];  // plain floats: always promoted to registers
  staticFor<LOADS>([&](auto ii) {
    constexpr int i = decltype(ii)::value;
    const float4 v = src[min(t + k1dThreads * i, max(total / 2 - 1, 0))];
    in[4 * i] = v.x;
    in[4 * i + 1] = v.y;
    in[4 * i + 2] = v.z;
    in[4 * i + 3] = v.w;
  });
  float4* l4 = reinterpret_cast<float4*>(lds);
  staticFor<LOADS>([&](auto ii) {
    constexpr int i = decltype(ii)::value;
    const int q = t + k1dThreads * i;
    if (q < total / 2) l4[q] = float4{in[4 * i], in[4 * i + 1], in[4 * i + 2], in[4 * i + 3]};
  });
  if ((total & 1) && t == 0)
    lds[total - 1] = reinterpret_cast<const float2*>(cplx + (size_t)b0 * 2 * RS)[total - 1];
  __syncthreads();

  // ROWS is a multiple of 64: g is the same for a whole wave, and says so
  const int row = t % ROWS, g = __builtin_amdgcn_readfirstlane(t / ROWS);
  c32* zrow = lds + row * RS;
  float* frow = reinterpret_cast<float*>(zrow);
  c32 zz[Q];
  if constexpr (G == 1) {
    // only the real parts of F[0] and F[H] reach a real result
    realFixupInverseFetch<H>(
        [&](auto kk) {
          constexpr int k = decltype(kk)::value;
          if constexpr (k == 0)
            return c32{zrow[0].x, zrow[H].x};
          else
            return zrow[k];
        },
        zz);
    regFFT<H, false>(zz);
    // private row, all of it in registers: store x[2j], x[2j+1]
    staticFor<Q>([&](auto jj) {
      constexpr int j = decltype(jj)::value;
      zrow[j] = zz[slot<Q>(j)];
    });
  } else if constexpr (G == 4) {
    // lane g takes z[4m + g]; E_g = IFFT(z[4m + g]), x[j + Q q] = sum_g i^(g q) w^(g j) E_g[j]
    auto pairFix = [&](auto kk, c32& zk, c32& zhk) __attribute__((always_inline)) {
      constexpr int k = decltype(kk)::value;
      const c32 a = zrow[k], bb = zrow[H - k];
      const c32 e = c32{a.x + bb.x, a.y - bb.y};
      const c32 d = c32{a.x - bb.x, a.y + bb.y};
      const c32 o = mulRoot<N, k, false>(d);
      zk = c32{e.x - o.y, e.y + o.x};
      zhk = c32{e.x + o.y, o.x - e.y};
    };
    if (g == 0) {
      const float f0 = zrow[0].x, fh = zrow[H].x;
      zz[0] = c32{f0 + fh, f0 - fh};
      staticFor<Q / 2 - 1>([&](auto mm) {
        constexpr int m = decltype(mm)::value + 1;  // z[4m] and z[H - 4m] = z[4(Q - m)]
        pairFix(std::integral_constant<int, 4 * m>{}, zz[m], zz[Q - m]);
      });
      const c32 a = zrow[H / 2];
      zz[Q / 2] = c32{2.0f * a.x, -2.0f * a.y};
    } else if (g == 2) {
      staticFor<Q / 2>([&](auto mm) {
        constexpr int m = decltype(mm)::value;      // z[4m+2] and z[H-4m-2] = z[4(Q-1-m)+2]
        pairFix(std::integral_constant<int, 4 * m + 2>{}, zz[m], zz[Q - 1 - m]);
      });
    } else if (g == 1) {
      staticFor<Q>([&](auto mm) {
        constexpr int m = decltype(mm)::value;      // own z[4m+1]; the pair's other half is lane 3's
        c32 drop;
        pairFix(std::integral_constant<int, 4 * m + 1>{}, zz[m], drop);
      });
    } else {
      staticFor<Q>([&](auto mm) {
        constexpr int m = decltype(mm)::value;      // own z[4m+3] = z[H - k], k = 4(Q-1-m)+1
        c32 drop;
        pairFix(std::integral_constant<int, 4 * (Q - 1 - m) + 1>{}, drop, zz[m]);
      });
    }
    regFFT<Q, false>(zz);
    // w^(g j), w = e^(2 pi i / H); exponents of H/2 and more are the negated lower half
    auto twist = [&](auto gg) __attribute__((always_inline)) {
      constexpr int GG = decltype(gg)::value;
      staticFor<Q>([&](auto jj) {
        constexpr int j = decltype(jj)::value;
        constexpr int ex = GG * j;
        const c32 val = zz[slot<Q>(j)];
        if constexpr (ex < H / 2) {
          zz[slot<Q>(j)] = mulRoot<H, ex, false>(val);
        } else {
          const c32 r = mulRoot<H, ex - H / 2, false>(val);
          zz[slot<Q>(j)] = c32{-r.x, -r.y};
        }
      });
    };
    if (g == 1) twist(std::integral_constant<int, 1>{});
    if (g == 2) twist(std::integral_constant<int, 2>{});
    if (g == 3) twist(std::integral_constant<int, 3>{});
    __syncthreads();  // all four lanes of a row have read it
    staticFor<Q>([&](auto jj) {
      constexpr int j = decltype(jj)::value;
      zrow[Q * g + j] = zz[slot<Q>(j)];
    });
  } else {
    auto pairFix = [&](auto kk, c32& zk, c32& zhk) __attribute__((always_inline)) {
      constexpr int k = decltype(kk)::value;
      const c32 a = zrow[k], bb = zrow[H - k];
      const c32 e = c32{a.x + bb.x, a.y - bb.y};
      const c32 d = c32{a.x - bb.x, a.y + bb.y};
      const c32 o = mulRoot<N, k, false>(d);
      zk = c32{e.x - o.y, e.y + o.x};
      zhk = c32{e.x + o.y, o.x - e.y};
    };
    if (g == 0) {
      const float f0 = zrow[0].x, fh = zrow[H].x;
      zz[0] = c32{f0 + fh, f0 - fh};
      staticFor<Q / 2 - 1>([&](auto mm) {
        constexpr int k = 2 * (decltype(mm)::value + 1);  // 2, 4, ..., H/2 - 2
        pairFix(std::integral_constant<int, k>{}, zz[k / 2], zz[(H - k) / 2]);
      });
      const c32 a = zrow[H / 2];
      zz[Q / 2] = c32{2.0f * a.x, -2.0f * a.y};
    } else {
      staticFor<Q / 2>([&](auto mm) {
        constexpr int k = 2 * decltype(mm)::value + 1;    // 1, 3, ..., H/2 - 1
        pairFix(std::integral_constant<int, k>{}, zz[(k - 1) / 2], zz[(H - k - 1) / 2]);
      });
    }
    regFFT<Q, false>(zz);
    if (g == 1) {
      staticFor<Q>([&](auto jj) {
        constexpr int j = decltype(jj)::value;
        zz[slot<Q>(j)] = mulRoot<H, j, false>(zz[slot<Q>(j)]);
      });
    }
    __syncthreads();  // both lanes of a row have read it
    // E as floats [0, H) of the row, w^j O as floats [H, N)
    staticFor<Q>([&](auto jj) {
      constexpr int j = decltype(jj)::value;
      reinterpret_cast<c32*>(frow + H * g)[j] = zz[slot<Q>(j)];
    });
  }
  __syncthreads();

  // ---- rows out, 16 bytes per store ----
  float4* dst = reinterpret_cast<float4*>(real + (size_t)b0 * N);
  for (int q = t; q < rows * (N / 4); q += k1dThreads) {
    const int r = q / (N / 4), c4 = q % (N / 4);
    const float* base = reinterpret_cast<const float*>(lds + r * RS);
    float4 o;
    if constexpr (G == 1) {
      o = float4{base[4 * c4], base[4 * c4 + 1], base[4 * c4 + 2], base[4 * c4 + 3]};
    } else if constexpr (G == 4) {
      // complex outputs jc, jc+1 with jc = 2 c4 = j + Q q: A = T0 + (-1)^q T2,
      // Bv = T1 + (-1)^q T3, x = A + i^q Bv
      const int jc = 2 * c4, q4 = jc / Q, f = 2 * (jc % Q);
      const float s2 = (q4 & 1) ? -1.0f : 1.0f;
      float av[4], bv[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        av[e] = base[f + e] + s2 * base[2 * (2 * Q) + f + e];
        bv[e] = base[2 * Q + f + e] + s2 * base[3 * (2 * Q) + f + e];
      }
      // i^q (bx, by): q=0 (bx, by), 1 (-by, bx), 2 (-bx, -by), 3 (by, -bx)
      const bool rot = q4 & 1;
      const float sg = (q4 == 0 || q4 == 3) ? 1.0f : -1.0f;   // sign of the first component
      const float sh = (q4 == 0 || q4 == 1) ? 1.0f : -1.0f;   // sign of the second component
      o = float4{av[0] + sg * (rot ? bv[1] : bv[0]), av[1] + sh * (rot ? bv[0] : bv[1]),
                 av[2] + sg * (rot ? bv[3] : bv[2]), av[3] + sh * (rot ? bv[2] : bv[3])};
    } else {
      const int f = (4 * c4) % H;
      const float sg = 4 * c4 < H ? 1.0f : -1.0f;
      o = float4{base[f] + sg * base[H + f], base[f + 1] + sg * base[H + f + 1],
                 base[f + 2] + sg * base[H + f + 2], base[f + 3] + sg * base[H + f + 3]};
    }
    streamStore(dst + q, o);
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
  if (N >= 8 && padL == 0 && sx == 1 && sb == N && ck == 2 && cb == N + 2 && aligned(real, 16) &&
      aligned(cplx, 16)) {
    const int rowsPerGroup = N <= 64 ? k1dThreads : k1dThreads / (N / 64);
    dim3 grid(ceilDiv(B, rowsPerGroup)), block(k1dThreads);
    if (N == 8) {
      if (forward)
        fft1dMidForward<8><<<grid, block, 0, s>>>(real, cplx, B);
      else
        fft1dMidInverse<8><<<grid, block, 0, s>>>(cplx, real, B);
    } else if (N == 16) {
      if (forward)
        fft1dMidForward<16><<<grid, block, 0, s>>>(real, cplx, B);
      else
        fft1dMidInverse<16><<<grid, block, 0, s>>>(cplx, real, B);
    } else if (N == 32) {
      if (forward)
        fft1dMidForward<32><<<grid, block, 0, s>>>(real, cplx, B);
      else
        fft1dMidInverse<32><<<grid, block, 0, s>>>(cplx, real, B);
    } else if (N == 64) {
      if (forward)
        fft1dMidForward<64><<<grid, block, 0, s>>>(real, cplx, B);
      else
        fft1dMidInverse<64><<<grid, block, 0, s>>>(cplx, real, B);
    } else if (N == 128) {
      if (forward)
        fft1dMidForward<128><<<grid, block, 0, s>>>(real, cplx, B);
      else
        fft1dMidInverse<128><<<grid, block, 0, s>>>(cplx, real, B);
    } else {
      if (forward)
        fft1dMidForward<256><<<grid, block, 0, s>>>(real, cplx, B);
      else
        fft1dMidInverse<256><<<grid, block, 0, s>>>(cplx, real, B);
    }
    return launchStatus();
  }
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
