// 2D real-to-complex / complex-to-real transforms for N in {8, 16, 32}
// (replaces fbfft2DVertical_{8,16,32} / fbifft2DVertical_{8,16,32},
// fbfft/FFT2D32.cuh:361-533).  Output layout cplx[b][ky][kx], ky = 0..N/2.
//
// Design (one wave64 per workgroup, no workgroup-wide synchronisation):
//   * T = N/2 lanes share a plane, so a wave carries P = 128/N planes.
//   * column pass: lane l owns columns 2l and 2l+1.  It loads them with 8-byte
//     loads (a wave instruction covers whole 4N-byte rows), runs two N/2-point
//     complex FFTs on the even/odd-row packing entirely in VGPRs and applies the
//     real-input fix-up; spectral rows 0 and N/2 (both real) travel packed as
//     one complex row.
//   * padded LDS transpose (row stride N + pad complex) hands lane l the whole
//     packed row l, 16 bytes per access.
//   * row pass: one N-point complex FFT per lane, again fully in VGPRs;
//     bit reversal is just register naming.
//   * the result goes back through LDS and leaves as one contiguous stream of
//     16-byte stores per wave; rows 0 and N/2 are unpacked on the way out.
// The inverse runs the same steps backwards.  Each plane crosses HBM exactly
// once in each direction: 4N^2 + 8N(N/2+1) bytes.
//
// PACKED variants keep the reference's packed spectrum format (the Unpack = false
// store of fbfft/FFT2D32.cuh:421-427 and the PackedInput = true core of :302-316):
// cplx is [B][N/2][N][2] and its row 0 holds F[0][kx] + i F[N/2][kx], the form the
// row travels in inside the kernel anyway, so the copy stages move N/2 plain rows.
#include "common.h"
#include "fft2d_core.h"
#include "fft_regs.h"

namespace fbfft_amd {
namespace {

template <int N, bool PACKED = false>
struct SmallCfg {
  static constexpr int H = N / 2;
  static constexpr int T = N / 2;          // lanes per plane
  static constexpr int P = 64 / T;         // planes per wave
  static constexpr int ROWS = PACKED ? H : H + 1;  // spectral rows of a plane in memory
  static constexpr int RS = PlaneCfg<N>::RS;  // LDS row stride (complex)
  static constexpr int PS = (H + 1) * RS + (N == 8 ? 2 : 0);  // LDS plane stride (complex)
  static constexpr int F4_PER_PLANE = ROWS * N / 2;        // float4 per spectrum plane
  static constexpr int ITERS = P * F4_PER_PLANE / 64;      // float4 per lane per wave
  static_assert(P * F4_PER_PLANE % 64 == 0, "copy loop must divide evenly");
  static_assert(RS % 2 == 0 && PS % 2 == 0, "rows must stay 16-byte aligned");
};

// FAST_REAL: real is [B][N][N] with unit x stride, even row/batch strides,
//            8-byte aligned base and zero padding -> 8-byte vector accesses.
// FAST_CPLX: each spectrum plane is contiguous and 16-byte aligned.
// GPW:       groups of P planes a wave processes (1 or 2).  With 2, the loads of
//            the second group are issued as soon as the first group's columns
//            have left the registers, so they fly under the first group's row
//            pass and stores: the wave pays the HBM latency once instead of twice.
template <int N, bool FAST_REAL, bool FAST_CPLX, int GPW, bool PACKED>
__global__ __launch_bounds__(64) void fft2dSmallForward(RealView real, CplxView cplx, int padL,
                                                        int padU) {
  using C = SmallCfg<N, PACKED>;
  constexpr int H = C::H, T = C::T, P = C::P, RS = C::RS, PS = C::PS;
  __shared__ __align__(16) c32 lds[P * PS];

  const int lane = threadIdx.x;
  const int pl = lane / T;
  const int l = lane % T;
  const int B = real.B;
  c32* plane = lds + pl * PS;

  auto load = [&](int b0, c32 (&z0)[H], c32 (&z1)[H]) __attribute__((always_inline)) {
    const int b = min(b0 + pl, B - 1);  // tail lanes redo the last plane and skip the store
    if constexpr (FAST_REAL) {
      const float2* src = reinterpret_cast<const float2*>(real.data + (size_t)b * real.sb) + l;
      const int rs2 = real.sy / 2;
      staticFor<H>([&](auto jj) {
        constexpr int j = decltype(jj)::value;
        float2 r0 = src[(size_t)(2 * j) * rs2];
        float2 r1 = src[(size_t)(2 * j + 1) * rs2];
        z0[j] = c32{r0.x, r1.x};
        z1[j] = c32{r0.y, r1.y};
      });
    } else {
      loadColumnsWindow<N>(real.data + (size_t)b * real.sb, real.sy, real.sx, real.h, real.w, padL,
                           padU, l, z0, z1);
    }
  };

  // copy out: (H+1) x N complex per plane, rows 0 and H unpacked from packed row 0
  // (FULL: every plane of the group exists, the common case - no per-store test)
  auto copyOutImpl = [&](int b0, auto fullTag) __attribute__((always_inline)) {
    constexpr bool FULL = decltype(fullTag)::value;
    staticFor<C::ITERS>([&](auto tt) {
      constexpr int t = decltype(tt)::value;
      // One iteration stores 64 / (N/2) consecutive spectral rows.  When none of
      // them is row 0 or N/2 of a plane (12 of the 17 iterations at N = 32) plane and
      // row are compile-time constants plus the lane's row within the iteration.
      constexpr int RPI = 64 / (N / 2);
      constexpr int R0 = RPI * t, pp0 = R0 / C::ROWS, r0 = R0 % C::ROWS;
      if constexpr ((PACKED || r0 >= 1) && r0 + RPI - 1 <= H - 1) {
        const int g = lane / (N / 2), xq = lane % (N / 2);
        const float4 v = ldsLoad4(lds + pp0 * PS + (r0 + g) * RS + 2 * xq);
        const int bo = b0 + pp0;
        if (FULL || bo < B) {
          if constexpr (FAST_CPLX) {
            streamStore(reinterpret_cast<float4*>(cplx.data + (size_t)bo * cplx.sb) + (r0 + g) * (N / 2) + xq, v);
          } else {
            float* o = cplx.data + (size_t)bo * cplx.sb + (size_t)(r0 + g) * cplx.sr +
                       (size_t)(2 * xq) * cplx.sc;
            *reinterpret_cast<float2*>(o) = float2{v.x, v.y};
            *reinterpret_cast<float2*>(o + cplx.sc) = float2{v.z, v.w};
          }
        }
        return;
      }
      const int q = lane + 64 * t;
      const int pp = q / C::F4_PER_PLANE;
      const int rem = q % C::F4_PER_PLANE;
      const int r = rem / (N / 2);
      const int kx = 2 * (rem % (N / 2));
      const c32* base = lds + pp * PS;
      float4 v;
      if (!PACKED && (r == 0 || r == H)) {
        c32 a0 = base[kx], a1 = base[kx + 1];
        c32 m0 = base[(N - kx) & (N - 1)], m1 = base[N - kx - 1];
        if (r == 0) {
          v = float4{0.5f * (a0.x + m0.x), 0.5f * (a0.y - m0.y), 0.5f * (a1.x + m1.x),
                     0.5f * (a1.y - m1.y)};
        } else {
          v = float4{0.5f * (a0.y + m0.y), 0.5f * (m0.x - a0.x), 0.5f * (a1.y + m1.y),
                     0.5f * (m1.x - a1.x)};
        }
      } else {
        v = ldsLoad4(base + r * RS + kx);
      }
      const int bo = b0 + pp;
      if (FULL || bo < B) {
        if constexpr (FAST_CPLX) {
          streamStore(reinterpret_cast<float4*>(cplx.data + (size_t)bo * cplx.sb) + rem, v);
        } else {
          float* o = cplx.data + (size_t)bo * cplx.sb + (size_t)r * cplx.sr + (size_t)kx * cplx.sc;
          *reinterpret_cast<float2*>(o) = float2{v.x, v.y};
          *reinterpret_cast<float2*>(o + cplx.sc) = float2{v.z, v.w};
        }
      }
    });
  };
  auto copyOut = [&](int b0) __attribute__((always_inline)) {
    if constexpr (N == 32 && GPW == 2) __builtin_amdgcn_s_setprio(0);
    if (b0 + P <= B)
      copyOutImpl(b0, std::true_type{});
    else
      copyOutImpl(b0, std::false_type{});
    if constexpr (N == 32 && GPW == 2) __builtin_amdgcn_s_setprio(2);
  };

  const int g0 = blockIdx.x * GPW * P;
  c32 za0[H], za1[H];
  load(g0, za0, za1);
  // A wave in its transform phases is given issue priority over the wave that shares
  // its SIMD while that one copies out.  Measured where every wave takes two groups
  // of 32 x 32 planes in one round: 21.80 -> 21.62 us; with one group per wave over
  // many rounds the same setting costs 2 %, at N = 16 and 8 it costs 5 % and 1 %, so
  // it is left alone there.
  if constexpr (N == 32 && GPW == 2) __builtin_amdgcn_s_setprio(2);
  columnPassForward<N>(za0, za1, plane, l);
  __syncthreads();
  c32 zb0[H], zb1[H];
  if constexpr (GPW == 2) load(g0 + P, zb0, zb1);
  rowPassInPlace<N, true>(plane, l);
  __syncthreads();
  copyOut(g0);
  if constexpr (GPW == 2) {
    __syncthreads();
    columnPassForward<N>(zb0, zb1, plane, l);
    __syncthreads();
    rowPassInPlace<N, true>(plane, l);
    __syncthreads();
    copyOut(g0 + P);
  }
}

__device__ __forceinline__ bool aligned16(const void* p) {
  return (reinterpret_cast<uintptr_t>(p) & 15) == 0;
}

template <int N, bool FAST_REAL, bool FAST_CPLX, int GPW, bool PACKED>
__global__ __launch_bounds__(64) void fft2dSmallInverse(CplxView cplx, RealView real, int padL,
                                                        int padU) {
  using C = SmallCfg<N, PACKED>;
  constexpr int H = C::H, T = C::T, P = C::P, RS = C::RS, PS = C::PS;
  __shared__ __align__(16) c32 lds[P * PS];

  const int lane = threadIdx.x;
  const int pl = lane / T;
  const int l = lane % T;
  const int B = real.B;
  c32* plane = lds + pl * PS;

  // spectra of one group, natural [row][kx] order, one float4 per lane per step
  float in[GPW][4 * C::ITERS];  // plain floats: always promoted to registers
  auto load = [&](auto gg, int b0) __attribute__((always_inline)) {
    constexpr int G = decltype(gg)::value;
    staticFor<C::ITERS>([&](auto tt) {
      constexpr int t = decltype(tt)::value;
      const int q = lane + 64 * t;
      const int pp = q / C::F4_PER_PLANE;
      const int rem = q % C::F4_PER_PLANE;
      const int bi = min(b0 + pp, B - 1);
      if constexpr (FAST_CPLX) {
        const float4 v = reinterpret_cast<const float4*>(cplx.data + (size_t)bi * cplx.sb)[rem];
        in[G][4 * t] = v.x;
        in[G][4 * t + 1] = v.y;
        in[G][4 * t + 2] = v.z;
        in[G][4 * t + 3] = v.w;
      } else {
        const int r = rem / (N / 2), kx = 2 * (rem % (N / 2));
        const float* o = cplx.data + (size_t)bi * cplx.sb + (size_t)r * cplx.sr + (size_t)kx * cplx.sc;
        float2 a = *reinterpret_cast<const float2*>(o);
        float2 c = *reinterpret_cast<const float2*>(o + cplx.sc);
        in[G][4 * t] = a.x;
        in[G][4 * t + 1] = a.y;
        in[G][4 * t + 2] = c.x;
        in[G][4 * t + 3] = c.y;
      }
    });
  };

  auto process = [&](auto gg, int b0) __attribute__((always_inline)) {
    constexpr int G = decltype(gg)::value;
    staticFor<C::ITERS>([&](auto tt) {
      constexpr int t = decltype(tt)::value;
      const int q = lane + 64 * t;
      const int pp = q / C::F4_PER_PLANE;
      const int rem = q % C::F4_PER_PLANE;
      *reinterpret_cast<float4*>(lds + pp * PS + (rem / (N / 2)) * RS + 2 * (rem % (N / 2))) =
          float4{in[G][4 * t], in[G][4 * t + 1], in[G][4 * t + 2], in[G][4 * t + 3]};
    });
    __syncthreads();
    // pack rows 0 and H into one complex row: Q = F0 + i*FH.  At kx = 0 only the real
    // parts are used, as in the reference (fbfft/FFT2D32.cuh:310-316).  Packed
    // operands arrive in that form.
    if constexpr (!PACKED) {
      c32* r0 = plane + 2 * l;
      const c32* rH = r0 + H * RS;
      float4 a = ldsLoad4(r0);
      float4 c = ldsLoad4(rH);
      float4 q = float4{a.x - c.y, a.y + c.x, a.z - c.w, a.w + c.z};
      if (l == 0) {
        q.x = a.x;
        q.y = c.x;
      }
      *reinterpret_cast<float4*>(r0) = q;
      __syncthreads();
    }
    rowPassInPlace<N, false>(plane, l);
    __syncthreads();
    c32 z0[H], z1[H];
    columnPassInverse<N>(plane, l, z0, z1);
    const int b = b0 + pl;
    if constexpr (FAST_REAL && N <= 16) {
      // Rows of 32 or 64 bytes: stored from the column layout, a wave instruction
      // would touch 16 or 8 cache lines with a fraction of each.  When the planes
      // of the group are contiguous in memory they go back through LDS instead and
      // leave as one stream of 16-byte stores.
      if (real.sy == N && real.sb == N * N && aligned16(real.data)) {
        __syncthreads();  // the spectra have been consumed
        float* stage = reinterpret_cast<float*>(lds);
        float* mine = stage + pl * N * N + 2 * l;
        staticFor<H>([&](auto jj) {
          constexpr int j = decltype(jj)::value;
          c32 a = z0[slot<H>(j)], c = z1[slot<H>(j)];
          *reinterpret_cast<float2*>(mine + (2 * j) * N) = float2{a.x, c.x};
          *reinterpret_cast<float2*>(mine + (2 * j + 1) * N) = float2{a.y, c.y};
        });
        __syncthreads();
        const int valid = min(P, B - b0) * (N * N / 4);  // float4 of the group's planes
        float4* dst = reinterpret_cast<float4*>(real.data + (size_t)b0 * (N * N));
        staticFor<P * N * N / 4 / 64>([&](auto ii) {
          constexpr int i = decltype(ii)::value;
          const int q = lane + 64 * i;
          if (q < valid) streamStore(dst + q, reinterpret_cast<const float4*>(stage)[q]);
        });
        return;
      }
    }
    if (b < B) {
      if constexpr (FAST_REAL) {
        float2* dst = reinterpret_cast<float2*>(real.data + (size_t)b * real.sb) + l;
        const int rs2 = real.sy / 2;
        staticFor<H>([&](auto jj) {
          constexpr int j = decltype(jj)::value;
          c32 a = z0[slot<H>(j)], c = z1[slot<H>(j)];
          streamStore(dst + (size_t)(2 * j) * rs2, float2{a.x, c.x});
          streamStore(dst + (size_t)(2 * j + 1) * rs2, float2{a.y, c.y});
        });
      } else {
        storeColumnsWindow<N>(real.data + (size_t)b * real.sb, real.sy, real.sx, real.h, real.w,
                              padL, padU, l, z0, z1, 1.0f);
      }
    }
  };

  const int g0 = blockIdx.x * GPW * P;
  constexpr std::integral_constant<int, 0> first{};
  load(first, g0);
  if constexpr (GPW == 2) {
    constexpr std::integral_constant<int, 1> second{};
    load(second, g0 + P);  // in flight while the first group is transformed
    process(first, g0);
    __syncthreads();
    process(second, g0 + P);
  } else {
    process(first, g0);
  }
}

// Two groups per wave pay off only when the launch would otherwise take between
// one and two rounds of resident waves: then the second round's load latency is
// exposed, and folding it into the first round's waves (with their loads already
// in flight) hides it.  Measured with operands that come from HBM (every launch on
// another set of buffers, more than 1 GiB in all), 32 x 32 R2C, us per launch
// paired / unpaired: 9216 planes 18.5 / 19.0, 10240 18.5 / 19.8, 12288 20.4 / 21.1,
// 14336 23.7 / 25.0, but 16384 (exactly two groups for every resident wave, all of
// them in step) 29.0 / 27.3; C2R 15.8 / 17.5, 16.6 / 18.4, 20.4 / 22.0, 24.0 / 25.0,
// 28.2 / 27.6.  16 x 16 (30720 planes resident): 32768 planes 14.2 / 16.4, 36864
// 16.7 / 17.6, 49152 21.8 / 21.9.  So waves pair up to 1.75 rounds; beyond that the
// hardware's own replacement of finished workgroups spreads loads and stores better.
// (On operands that stay in the last-level cache pairing is also ahead at 16384
// planes, 21.7 against 22.5 us.)
template <int N>
bool pairGroups(int groups) {
  constexpr int ldsBytes = SmallCfg<N>::P * SmallCfg<N>::PS * (int)sizeof(c32);
  constexpr int wavesPerCU = (160 * 1024 / ldsBytes) < 32 ? (160 * 1024 / ldsBytes) : 32;
  const long slots = (long)computeUnits() * wavesPerCU;
  return groups > slots && 4L * groups <= 7 * slots;
}

bool fastReal(int N, const RealView& r, int padL, int padU) {
  return padL == 0 && padU == 0 && r.h == N && r.w == N && r.sx == 1 && r.sy % 2 == 0 &&
         r.sb % 2 == 0 && aligned(r.data, 8);
}

bool fastCplx(int N, const CplxView& c) {
  return c.sc == 2 && c.sr == 2 * N && c.sb % 4 == 0 && aligned(c.data, 16);
}

// runs f(std::bool_constant<a>{}, std::bool_constant<b>{}) for the run-time pair (a, b)
template <typename F>
void withFlags(bool a, bool b, F&& f) {
  if (a && b) f(std::true_type{}, std::true_type{});
  else if (a) f(std::true_type{}, std::false_type{});
  else if (b) f(std::false_type{}, std::true_type{});
  else f(std::false_type{}, std::false_type{});
}

template <int N, bool PACKED>
int launchForward(const RealView& real, const CplxView& cplx, int padL, int padU, hipStream_t s) {
  using C = SmallCfg<N, PACKED>;
  const int groups = ceilDiv(real.B, C::P);
  dim3 block(64);
  withFlags(fastReal(N, real, padL, padU), fastCplx(N, cplx), [&](auto fr, auto fc) {
    constexpr bool FR = decltype(fr)::value, FC = decltype(fc)::value;
    if (pairGroups<N>(groups))
      fft2dSmallForward<N, FR, FC, 2, PACKED><<<dim3(ceilDiv(groups, 2)), block, 0, s>>>(real, cplx, padL, padU);
    else
      fft2dSmallForward<N, FR, FC, 1, PACKED><<<dim3(groups), block, 0, s>>>(real, cplx, padL, padU);
  });
  return launchStatus();
}

template <int N, bool PACKED>
int launchInverse(const CplxView& cplx, const RealView& real, int padL, int padU, hipStream_t s) {
  using C = SmallCfg<N, PACKED>;
  const int groups = ceilDiv(real.B, C::P);
  dim3 block(64);
  withFlags(fastReal(N, real, padL, padU), fastCplx(N, cplx), [&](auto fr, auto fc) {
    constexpr bool FR = decltype(fr)::value, FC = decltype(fc)::value;
    if (pairGroups<N>(groups))
      fft2dSmallInverse<N, FR, FC, 2, PACKED><<<dim3(ceilDiv(groups, 2)), block, 0, s>>>(cplx, real, padL, padU);
    else
      fft2dSmallInverse<N, FR, FC, 1, PACKED><<<dim3(groups), block, 0, s>>>(cplx, real, padL, padU);
  });
  return launchStatus();
}

}  // namespace

// packed: cplx is [B][N/2][N][2] with rows 0 and N/2 of the spectrum packed in row 0
int launchFft2dSmallForward(int N, const RealView& real, const CplxView& cplx, int padL, int padU,
                            hipStream_t s, bool packed) {
  if (real.B <= 0) return FBFFT_SUCCESS;
  switch (N) {
    case 8: return packed ? launchForward<8, true>(real, cplx, padL, padU, s)
                          : launchForward<8, false>(real, cplx, padL, padU, s);
    case 16: return packed ? launchForward<16, true>(real, cplx, padL, padU, s)
                           : launchForward<16, false>(real, cplx, padL, padU, s);
    case 32: return packed ? launchForward<32, true>(real, cplx, padL, padU, s)
                           : launchForward<32, false>(real, cplx, padL, padU, s);
  }
  return FBFFT_UNSUPPORTED_SIZE;
}

int launchFft2dSmallInverse(int N, const CplxView& cplx, const RealView& real, int padL, int padU,
                            hipStream_t s, bool packed) {
  if (real.B <= 0) return FBFFT_SUCCESS;
  switch (N) {
    case 8: return packed ? launchInverse<8, true>(cplx, real, padL, padU, s)
                          : launchInverse<8, false>(cplx, real, padL, padU, s);
    case 16: return packed ? launchInverse<16, true>(cplx, real, padL, padU, s)
                           : launchInverse<16, false>(cplx, real, padL, padU, s);
    case 32: return packed ? launchInverse<32, true>(cplx, real, padL, padU, s)
                           : launchInverse<32, false>(cplx, real, padL, padU, s);
  }
  return FBFFT_UNSUPPORTED_SIZE;
}

}  // namespace fbfft_amd
