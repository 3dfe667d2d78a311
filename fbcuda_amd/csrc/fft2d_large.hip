// 2D real-to-complex / complex-to-real transforms for N in {64, 128} in ONE
// kernel and one pass over HBM.  The reference needs two kernels and a scratch
// round trip for these sizes (fbfft/FBFFT2D-inl.cuh:230-444,
// fbfft/FBIFFT2D-inl.cuh:252-521).  Output layout cplx[b][kx][ky], kx = 0..N/2:
// the Hermitian-halved axis is the horizontal frequency and the plane is stored
// transposed, as the reference's second pass leaves it.
//
// One workgroup owns one plane, which stays in LDS between the passes (one
// buffer, reused by every stage):
//   1. coalesced 16-byte loads of the real plane into LDS, rows padded by 4 floats;
//   2. row pass: lane y turns row y (N reals) into N/2 packed complex values and
//      runs an N/2-point complex FFT in VGPRs plus the real-input fix-up;
//      columns kx = 0 and kx = N/2 (both real along y) travel packed as one;
//   3. the result is written back transposed ([kx][y], odd row stride: no bank
//      conflicts either way);
//   4. column pass: each N-point column FFT is split over G lanes (G = 2 for 64,
//      G = 4 for 128; for 128 G is the wave index): lane g forms the radix-G
//      decimation-in-frequency sums for its residue straight from LDS, applies
//      W_N^(g*j) from an LDS copy of the twiddle table and finishes with a
//      32-point FFT in VGPRs;
//   5. results return to LDS as [kx][ky] and leave as one contiguous stream of
//      16-byte stores; the packed column is unpacked on the way out.
// The inverse runs the same steps backwards and crops on store.
#include "common.h"
#include "fft_lds.h"
#include "fft_regs.h"

namespace fbfft_amd {
namespace {

template <int N>
struct LargeCfg {
  static constexpr int H = N / 2;
  static constexpr int G = (N == 64) ? 2 : 4;   // lanes per column FFT
  static constexpr int L = N / G;               // points per lane in the column pass (32)
  static constexpr int THREADS = H * G;         // 64 or 256
  static constexpr int RSF = N + 4;             // real-plane row stride in floats (16-byte rows)
  static constexpr int RSI = (N == 128) ? N + 2 : N + 4;  // forward input stage: for 128 the rows are
                                                // read as complex pairs by 2 lanes each, odd
                                                // complex stride = no bank conflicts
  static constexpr int GR = (N == 128) ? 2 : 1; // lanes per row transform
  static constexpr int CS = N + 1;              // [kx][y|ky] row stride in complex
  static constexpr int YS = H + 1;              // [y][kx] row stride in complex (inverse)
  static constexpr int BUF_FLOATS =
      (N * RSF > 2 * H * CS ? (N * RSF > 2 * N * YS ? N * RSF : 2 * N * YS)
                            : (2 * H * CS > 2 * N * YS ? 2 * H * CS : 2 * N * YS));
  static constexpr int F4_REAL = N * N / 4;           // float4 per real plane
  static constexpr int F4_CPLX = (H + 1) * N / 2;     // float4 per spectrum plane
};

template <int N, bool FAST_REAL, bool FAST_CPLX>
__global__ __launch_bounds__(LargeCfg<N>::THREADS) void fft2dLargeForward(RealView real,
                                                                         CplxView cplx, int padL,
                                                                         int padU) {
  using C = LargeCfg<N>;
  constexpr int H = C::H, G = C::G, L = C::L, THREADS = C::THREADS, CS = C::CS;
  __shared__ __align__(16) float buf[C::BUF_FLOATS];
  __shared__ __align__(8) c32 tw[256];
  const int t = threadIdx.x;
  const int b = blockIdx.x;
  fillTwiddles<true>(tw, t, THREADS);

  constexpr int RSI = C::RSI;
  // ---- 1. real plane -> LDS [y][x] ----
  if constexpr (FAST_REAL) {
    const float4* src = reinterpret_cast<const float4*>(real.data + (size_t)b * real.sb);
    const int rs4 = real.sy / 4;
    staticFor<C::F4_REAL / THREADS>([&](auto ii) {
      constexpr int i = decltype(ii)::value;
      const int q = t + THREADS * i;
      const float4 v = src[(size_t)(q / (N / 4)) * rs4 + q % (N / 4)];
      float* d = buf + (q / (N / 4)) * RSI + 4 * (q % (N / 4));
      if constexpr (RSI % 4 == 0) {
        *reinterpret_cast<float4*>(d) = v;
      } else {
        *reinterpret_cast<float2*>(d) = float2{v.x, v.y};
        *reinterpret_cast<float2*>(d + 2) = float2{v.z, v.w};
      }
    });
  } else {
    // Windowed plane (implicit zero padding, any strides): a lane keeps its column
    // and walks down the rows.  Loads go out in batches of 16 at addresses clamped
    // into the window, with no branch between them, and samples outside the window
    // are zeroed when they are parked in LDS; batches below the window's last row
    // load nothing.
    const float* src = real.data + (size_t)b * real.sb;
    const int yEnd = min(N, padU + real.h);
    // rows that start on 16-byte boundaries and a window whose left edge and width are
    // multiples of 4 (contiguous 60 x 60 planes, say) move as float4 the same way
    const bool vec = real.sx == 1 && ((real.sy | real.sb | padL | real.w) & 3) == 0 &&
                     (reinterpret_cast<uintptr_t>(real.data) & 15) == 0;
    if (vec) {
      constexpr int GPR = N / 4;           // float4 per row
      constexpr int RPI4 = THREADS / GPR;  // rows per step
      constexpr int STEPS = N / RPI4;      // 16
      constexpr int HALF = STEPS / 2;
      const int xg = t % GPR, yb = t / GPR;
      const int xs = 4 * xg - padL;
      const bool xin = (unsigned)xs < (unsigned)real.w;
      const float* colp = src + min(max(xs, 0), real.w - 4);
#pragma unroll
      for (int j0 = 0; j0 < STEPS; j0 += HALF) {
        float4 v[HALF];
        if (j0 * RPI4 < yEnd) {
#pragma unroll
          for (int j = 0; j < HALF; ++j) {
            const int ys = min(max(yb + RPI4 * (j0 + j) - padU, 0), real.h - 1);
            v[j] = *reinterpret_cast<const float4*>(colp + (size_t)ys * real.sy);
          }
        }
#pragma unroll
        for (int j = 0; j < HALF; ++j) {
          const int y = yb + RPI4 * (j0 + j);
          const bool ok = j0 * RPI4 < yEnd && xin && (unsigned)(y - padU) < (unsigned)real.h;
          const float4 o = ok ? v[j] : float4{0.f, 0.f, 0.f, 0.f};
          float* d = buf + y * RSI + 4 * xg;
          if constexpr (RSI % 4 == 0) {
            *reinterpret_cast<float4*>(d) = o;
          } else {
            *reinterpret_cast<float2*>(d) = float2{o.x, o.y};
            *reinterpret_cast<float2*>(d + 2) = float2{o.z, o.w};
          }
        }
      }
    } else {
    constexpr int RPI = THREADS / N;   // rows per step of the walk
    constexpr int BATCH = 16;
    const int x = t % N, yb = t / N;
    const int xs = x - padL;
    const bool xin = (unsigned)xs < (unsigned)real.w;
    const float* colp = src + (size_t)min(max(xs, 0), real.w - 1) * real.sx;
#pragma unroll
    for (int i0 = 0; i0 < N / RPI; i0 += BATCH) {
      if (i0 * RPI < yEnd) {
        float v[BATCH];
#pragma unroll
        for (int j = 0; j < BATCH; ++j) {
          const int ys = min(max(yb + RPI * (i0 + j) - padU, 0), real.h - 1);
          v[j] = colp[(size_t)ys * real.sy];
        }
#pragma unroll
        for (int j = 0; j < BATCH; ++j) {
          const int y = yb + RPI * (i0 + j);
          buf[y * RSI + x] = (xin && (unsigned)(y - padU) < (unsigned)real.h) ? v[j] : 0.0f;
        }
      } else {
#pragma unroll
        for (int j = 0; j < BATCH; ++j) buf[(yb + RPI * (i0 + j)) * RSI + x] = 0.0f;
      }
    }
    }
  }
  __syncthreads();

  c32* cb = reinterpret_cast<c32*>(buf);
  if constexpr (C::GR == 1) {
    // ---- 2. row pass: lane y, N reals -> H packed complex ----
    c32 z[H];
    if (t < N) {
      const float* row = buf + t * RSI;
      staticFor<H / 2>([&](auto mm) {
        constexpr int m = decltype(mm)::value;
        float4 v = *reinterpret_cast<const float4*>(row + 4 * m);
        z[2 * m] = c32{v.x, v.y};
        z[2 * m + 1] = c32{v.z, v.w};
      });
    }
    __syncthreads();  // every row is in registers: the buffer may be overwritten
    if (t < N) {
      regFFT<H, true>(z);
      // ---- 3. fix-up fused with the transposed write: [kx][y] ----
      realFixupForwardEmit<H>(z, [&](auto kk, c32 val) {
        constexpr int k = decltype(kk)::value;
        cb[k * CS + t] = val;
      });
    }
  } else {
    // ---- 2. row pass split over two lanes: lane (y, gr) gets Z[2k + gr] of the
    // H-point transform of row y; gr is uniform per wave ----
    const int y = t % N, gr = t / N;
    constexpr int LR = H / 2;
    c32 v[LR];
    splitFFT<H, 2, true>(reinterpret_cast<const c32*>(buf + y * RSI), gr, tw, v);
    __syncthreads();  // every row consumed: the buffer may be overwritten
    // ---- 3. fix-up: bins k' and H-k' have the same parity, so each lane finishes
    // its own half; twiddles are compile-time in both branches ----
    auto pairOut = [&](auto kp, c32 a, c32 bq) {
      constexpr int k = decltype(kp)::value;  // bin k pairs with H-k
      c32 fk, fhk;
      realPairForward<N, k>(a, bq, fk, fhk);
      cb[k * CS + y] = fk;
      cb[(H - k) * CS + y] = fhk;
    };
    if (gr == 0) {
      c32 z0 = v[0];
      cb[y] = c32{z0.x + z0.y, z0.x - z0.y};
      staticFor<LR / 2 - 1>([&](auto kk) {
        constexpr int k = decltype(kk)::value + 1;  // bins 2k and H-2k
        pairOut(std::integral_constant<int, 2 * k>{}, v[slot<LR>(k)], v[slot<LR>(LR - k)]);
      });
      c32 m = v[slot<LR>(LR / 2)];  // bin H/2
      cb[(H / 2) * CS + y] = c32{m.x, -m.y};
    } else {
      staticFor<LR / 2>([&](auto kk) {
        constexpr int k = decltype(kk)::value;  // bins 2k+1 and H-2k-1
        pairOut(std::integral_constant<int, 2 * k + 1>{}, v[slot<LR>(k)], v[slot<LR>(LR - 1 - k)]);
      });
    }
  }
  __syncthreads();

  // ---- 4. column pass ----
  const int col = t % H, g = t / H;
  c32 v[L];
  splitFFT<N, G, true>(cb + col * CS, g, tw, v);
  __syncthreads();  // all columns consumed
  // ---- 5. [kx][ky] back to LDS ----
  staticFor<L>([&](auto kk) {
    constexpr int k = decltype(kk)::value;
    cb[col * CS + G * k + g] = v[slot<L>(k)];
  });
  __syncthreads();

  // ---- copy out (H+1) x N complex; rows 0 and H come from packed row 0 ----
  constexpr int ITERS = (C::F4_CPLX + THREADS - 1) / THREADS;
  staticFor<ITERS>([&](auto ii) {
    constexpr int i = decltype(ii)::value;
    const int q = t + THREADS * i;
    if (q < C::F4_CPLX) {
      const int r = q / (N / 2);
      const int ky = 2 * (q % (N / 2));
      float4 o;
      if (r == 0 || r == H) {
        c32 a0 = cb[ky], a1 = cb[ky + 1];
        c32 m0 = cb[(N - ky) & (N - 1)], m1 = cb[N - ky - 1];
        if (r == 0)
          o = float4{0.5f * (a0.x + m0.x), 0.5f * (a0.y - m0.y), 0.5f * (a1.x + m1.x),
                     0.5f * (a1.y - m1.y)};
        else
          o = float4{0.5f * (a0.y + m0.y), 0.5f * (m0.x - a0.x), 0.5f * (a1.y + m1.y),
                     0.5f * (m1.x - a1.x)};
      } else {
        c32 a0 = cb[r * CS + ky], a1 = cb[r * CS + ky + 1];
        o = float4{a0.x, a0.y, a1.x, a1.y};
      }
      if constexpr (FAST_CPLX) {
        streamStore(reinterpret_cast<float4*>(cplx.data + (size_t)b * cplx.sb) + q, o);
      } else {
        float* dst = cplx.data + (size_t)b * cplx.sb + (size_t)r * cplx.sr + (size_t)ky * cplx.sc;
        *reinterpret_cast<float2*>(dst) = float2{o.x, o.y};
        *reinterpret_cast<float2*>(dst + cplx.sc) = float2{o.z, o.w};
      }
    }
  });
}

template <int N, bool FAST_REAL, bool FAST_CPLX>
__global__ __launch_bounds__(LargeCfg<N>::THREADS) void fft2dLargeInverse(CplxView cplx,
                                                                         RealView real, int padL,
                                                                         int padU) {
  using C = LargeCfg<N>;
  constexpr int H = C::H, G = C::G, L = C::L, THREADS = C::THREADS, RSF = C::RSF, CS = C::CS,
                YS = C::YS;
  __shared__ __align__(16) float buf[C::BUF_FLOATS];
  __shared__ __align__(8) c32 tw[256];
  const int t = threadIdx.x;
  const int b = blockIdx.x;
  fillTwiddles<false>(tw, t, THREADS);
  c32* cb = reinterpret_cast<c32*>(buf);

  // ---- copy in [kx][ky].  All loads are issued before any is consumed (no load
  // sits behind a branch or a barrier); the lanes that hold row 0 also fetch row H
  // and store the fold Z = F0 + i*FH. ----
  static_assert(H * (N / 2) % THREADS == 0, "rows 0..H-1 divide evenly over the lanes");
  constexpr int ITERS = H * (N / 2) / THREADS;
  auto fetch4 = [&](int r, int ky, int q) {
    if constexpr (FAST_CPLX) {
      return reinterpret_cast<const float4*>(cplx.data + (size_t)b * cplx.sb)[q];
    } else {
      const float* src = cplx.data + (size_t)b * cplx.sb + (size_t)r * cplx.sr + (size_t)ky * cplx.sc;
      float2 a = *reinterpret_cast<const float2*>(src);
      float2 c = *reinterpret_cast<const float2*>(src + cplx.sc);
      return float4{a.x, a.y, c.x, c.y};
    }
  };
  float4 in[ITERS];
  staticFor<ITERS>([&](auto ii) {
    constexpr int i = decltype(ii)::value;
    const int q = t + THREADS * i;
    in[i] = fetch4(q / (N / 2), 2 * (q % (N / 2)), q);
  });
  {
    const int tq = t % (N / 2);  // lanes beyond the first N/2 fetch a duplicate they ignore
    const float4 u = fetch4(H, 2 * tq, H * (N / 2) + tq);
    if (t < N / 2) in[0] = float4{in[0].x - u.y, in[0].y + u.x, in[0].z - u.w, in[0].w + u.z};
  }
  staticFor<ITERS>([&](auto ii) {
    constexpr int i = decltype(ii)::value;
    const int q = t + THREADS * i;
    const int r = q / (N / 2);
    const int ky = 2 * (q % (N / 2));
    cb[r * CS + ky] = c32{in[i].x, in[i].y};
    cb[r * CS + ky + 1] = c32{in[i].z, in[i].w};
  });
  __syncthreads();

  // ---- column pass (inverse) ----
  const int col = t % H, g = t / H;
  c32 v[L];
  splitFFT<N, G, false>(cb + col * CS, g, tw, v);
  __syncthreads();
  // [y][kx]
  staticFor<L>([&](auto kk) {
    constexpr int k = decltype(kk)::value;
    cb[(G * k + g) * YS + col] = v[slot<L>(k)];
  });
  __syncthreads();

  if constexpr (THREADS == N) {
    // ---- row pass (inverse): lane y ----
    c32 z[H];
    {
      const c32* row = cb + t * YS;
      realFixupInverseFetch<H>([&](auto kk) { return row[decltype(kk)::value]; }, z);
      regFFT<H, false>(z);
    }
    __syncthreads();
    {
      float* row = buf + t * RSF;
      staticFor<H / 2>([&](auto mm) {
        constexpr int m = decltype(mm)::value;
        c32 a = z[slot<H>(2 * m)], c = z[slot<H>(2 * m + 1)];
        *reinterpret_cast<float4*>(row + 4 * m) = float4{a.x, a.y, c.x, c.y};
      });
    }
    __syncthreads();

    // ---- copy out, cropped to the window real covers ----
    if constexpr (FAST_REAL) {
      float4* dst = reinterpret_cast<float4*>(real.data + (size_t)b * real.sb);
      const int rs4 = real.sy / 4;
      staticFor<C::F4_REAL / THREADS>([&](auto ii) {
        constexpr int i = decltype(ii)::value;
        const int q = t + THREADS * i;
        const int y = q / (N / 4), x4 = q % (N / 4);
        streamStore(dst + (size_t)y * rs4 + x4, *reinterpret_cast<const float4*>(buf + y * RSF + 4 * x4));
      });
    } else {
      // a lane keeps its column and walks down the rows of the window
      constexpr int RPI = THREADS / N;
      const int x = t % N, xs = x - padL;
      if ((unsigned)xs < (unsigned)real.w) {
        float* colp = real.data + (size_t)b * real.sb + (size_t)xs * real.sx;
        const int yEnd = min(N, padU + real.h);
#pragma unroll 8
        for (int y = padU + t / N; y < yEnd; y += RPI)
          colp[(size_t)(y - padU) * real.sy] = buf[y * RSF + x];
      }
    }
  } else {
    // ---- row pass (inverse) over two lanes per row y.  The H-point inverse
    // transform of z splits by the parity of its input index: lane g takes
    // z[2m + g], whose real-input fix-up pairs (k, H - k) have the same parity, so
    // neither lane repeats the other's fix-up.  With E = IFFT(z even), O = IFFT(z odd)
    // the result is x[j] = E[j] + w^j O[j], x[j + H/2] = E[j] - w^j O[j], w = e^{2 pi i/H}.
    // Lane 1 scales its half by w^j; the sum and difference are formed on the way
    // out of LDS.  g is the same for a whole wave. ----
    static_assert(THREADS == 2 * N, "two lanes per row");
    constexpr int Q = H / 2;  // points per lane
    const int y = t % N, g = t / N;
    c32 zz[Q];
    {
      const c32* row = cb + y * YS;
      auto pairFix = [&](auto kk, c32& zk, c32& zhk) __attribute__((always_inline)) {
        constexpr int k = decltype(kk)::value;
        const c32 a = row[k], bb = row[H - k];
        const c32 e = c32{a.x + bb.x, a.y - bb.y};
        const c32 d = c32{a.x - bb.x, a.y + bb.y};
        const c32 o = mulRoot<N, k, false>(d);
        zk = c32{e.x - o.y, e.y + o.x};
        zhk = c32{e.x + o.y, o.x - e.y};
      };
      if (g == 0) {
        const c32 p0 = row[0];
        zz[0] = c32{p0.x + p0.y, p0.x - p0.y};
        staticFor<Q / 2 - 1>([&](auto mm) {
          constexpr int k = 2 * (decltype(mm)::value + 1);  // 2, 4, ..., H/2 - 2
          pairFix(std::integral_constant<int, k>{}, zz[k / 2], zz[(H - k) / 2]);
        });
        const c32 a = row[H / 2];
        zz[Q / 2] = c32{2.0f * a.x, -2.0f * a.y};
      } else {
        staticFor<Q / 2>([&](auto mm) {
          constexpr int k = 2 * decltype(mm)::value + 1;    // 1, 3, ..., H/2 - 1
          pairFix(std::integral_constant<int, k>{}, zz[(k - 1) / 2], zz[(H - k - 1) / 2]);
        });
      }
    }
    regFFT<Q, false>(zz);
    if (g == 1) {
      staticFor<Q>([&](auto jj) {
        constexpr int j = decltype(jj)::value;
        zz[slot<Q>(j)] = mulRoot<H, j, false>(zz[slot<Q>(j)]);
      });
    }
    __syncthreads();
    {
      // row y of the staging buffer: E as floats [0, H), w^j O as floats [H, N)
      float* row = buf + y * RSF + H * g;
      staticFor<Q / 2>([&](auto mm) {
        constexpr int m = decltype(mm)::value;
        c32 a = zz[slot<Q>(2 * m)], c = zz[slot<Q>(2 * m + 1)];
        *reinterpret_cast<float4*>(row + 4 * m) = float4{a.x, a.y, c.x, c.y};
      });
    }
    __syncthreads();

    // ---- copy out, cropped to the window real covers: real samples 2j, 2j+1 are
    // (re, im) of x[j] ----
    if constexpr (FAST_REAL) {
      float4* dst = reinterpret_cast<float4*>(real.data + (size_t)b * real.sb);
      const int rs4 = real.sy / 4;
      staticFor<C::F4_REAL / THREADS>([&](auto ii) {
        constexpr int i = decltype(ii)::value;
        const int q = t + THREADS * i;
        const int yy = q / (N / 4), x4 = q % (N / 4);
        const int f = (4 * x4) % H;  // float offset of E[j], j = 2*x4 mod H/2
        const float4 e = *reinterpret_cast<const float4*>(buf + yy * RSF + f);
        const float4 w = *reinterpret_cast<const float4*>(buf + yy * RSF + H + f);
        const float sg = 4 * x4 < H ? 1.0f : -1.0f;
        streamStore(dst + (size_t)yy * rs4 + x4,
                    float4{e.x + sg * w.x, e.y + sg * w.y, e.z + sg * w.z, e.w + sg * w.w});
      });
    } else {
      // a lane keeps its column and walks down the rows of the window
      constexpr int RPI = THREADS / N;
      const int x = t % N, xs = x - padL;
      if ((unsigned)xs < (unsigned)real.w) {
        float* colp = real.data + (size_t)b * real.sb + (size_t)xs * real.sx;
        const int yEnd = min(N, padU + real.h);
        const float sg = x < H ? 1.0f : -1.0f;
        const float* e = buf + x % H;
#pragma unroll 8
        for (int yy = padU + t / N; yy < yEnd; yy += RPI)
          colp[(size_t)(yy - padU) * real.sy] = e[yy * RSF] + sg * e[yy * RSF + H];
      }
    }
  }
}

bool fastReal(int N, const RealView& r, int padL, int padU) {
  return padL == 0 && padU == 0 && r.h == N && r.w == N && r.sx == 1 && r.sy % 4 == 0 &&
         r.sb % 4 == 0 && aligned(r.data, 16);
}

bool fastCplx(int N, const CplxView& c) {
  return c.sc == 2 && c.sr == 2 * N && c.sb % 4 == 0 && aligned(c.data, 16);
}

template <int N>
int launchForward(const RealView& real, const CplxView& cplx, int padL, int padU, hipStream_t s) {
  dim3 grid(real.B), block(LargeCfg<N>::THREADS);
  const bool fr = fastReal(N, real, padL, padU), fc = fastCplx(N, cplx);
  if (fr && fc)
    fft2dLargeForward<N, true, true><<<grid, block, 0, s>>>(real, cplx, padL, padU);
  else if (fc)
    fft2dLargeForward<N, false, true><<<grid, block, 0, s>>>(real, cplx, padL, padU);
  else if (fr)
    fft2dLargeForward<N, true, false><<<grid, block, 0, s>>>(real, cplx, padL, padU);
  else
    fft2dLargeForward<N, false, false><<<grid, block, 0, s>>>(real, cplx, padL, padU);
  return launchStatus();
}

template <int N>
int launchInverse(const CplxView& cplx, const RealView& real, int padL, int padU, hipStream_t s) {
  dim3 grid(real.B), block(LargeCfg<N>::THREADS);
  const bool fr = fastReal(N, real, padL, padU), fc = fastCplx(N, cplx);
  if (fr && fc)
    fft2dLargeInverse<N, true, true><<<grid, block, 0, s>>>(cplx, real, padL, padU);
  else if (fc)
    fft2dLargeInverse<N, false, true><<<grid, block, 0, s>>>(cplx, real, padL, padU);
  else if (fr)
    fft2dLargeInverse<N, true, false><<<grid, block, 0, s>>>(cplx, real, padL, padU);
  else
    fft2dLargeInverse<N, false, false><<<grid, block, 0, s>>>(cplx, real, padL, padU);
  return launchStatus();
}

}  // namespace

int launchFft2dLargeForward(int N, const RealView& real, const CplxView& cplx, int padL, int padU,
                            hipStream_t s) {
  if (real.B <= 0) return FBFFT_SUCCESS;
  if (N == 64) return launchForward<64>(real, cplx, padL, padU, s);
  if (N == 128) return launchForward<128>(real, cplx, padL, padU, s);
  return FBFFT_UNSUPPORTED_SIZE;
}

int launchFft2dLargeInverse(int N, const CplxView& cplx, const RealView& real, int padL, int padU,
                            hipStream_t s) {
  if (real.B <= 0) return FBFFT_SUCCESS;
  if (N == 64) return launchInverse<64>(cplx, real, padL, padU, s);
  if (N == 128) return launchInverse<128>(cplx, real, padL, padU, s);
  return FBFFT_UNSUPPORTED_SIZE;
}

}  // namespace fbfft_amd
