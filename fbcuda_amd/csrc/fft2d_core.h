// Per-plane passes of the N <= 32 2D transforms, shared by the stand-alone
// kernels and by the fused tiled convolution.  A plane is handled by T = N/2
// lanes of one wave; lane l owns columns 2l, 2l+1 in the column pass and packed
// spectral row l in the row pass.  The plane buffer in LDS holds N/2 (+1) rows of
// N complex with row stride N + 2 (rows stay 16-byte aligned and consecutive rows
// start 4 banks apart, so 16-byte accesses by the lanes of a plane do not
// conflict).  Packed row 0 carries spectral rows 0 and N/2 (both real along the
// column axis) as real and imaginary part.  Callers place the barriers.
#pragma once

#include "common.h"
#include "fft_regs.h"

namespace fbfft_amd {

template <int N>
struct PlaneCfg {
  static constexpr int H = N / 2;
  static constexpr int T = N / 2;     // lanes per plane
  static constexpr int RS = N + 2;    // LDS row stride (complex)
};

__device__ __forceinline__ float4 ldsLoad4(const c32* p) {
  return *reinterpret_cast<const float4*>(p);
}
__device__ __forceinline__ void ldsStore4(c32* p, c32 a, c32 b) {
  *reinterpret_cast<float4*>(p) = float4{a.x, a.y, b.x, b.y};
}

// Two columns of a real plane through a bounds-checked strided view:
// z[j] = (X[2j][x], X[2j+1][x]) for x = 2l and 2l+1, zero outside the window
// (the padding rule of MemoryAccess.cuh:19-25).  Every load is issued
// unconditionally at an address clamped into the window and the value is zeroed
// afterwards, so the 2N loads of a lane are all in flight together and no branch
// separates them; the window must not be empty.  Row terms are wave-uniform.
// PAIRS = 0: one 4-byte load per sample, any strides.  PAIRS = 1: the caller
// guarantees windowMovesAsPairs() - rows on 8-byte boundaries, even left edge and
// width - so the lane's two columns are one 8-byte word per row, inside or outside
// the window together.  PAIRS = 2: decided here, per lane (the planes of a wave
// disagree only when the plane stride is odd; both paths then run under their masks).
__host__ __device__ __forceinline__ bool windowMovesAsPairs(const float* src, long sy, long sx,
                                                            int w, int padL) {
  return sx == 1 && ((sy | padL | w) & 1) == 0 && (reinterpret_cast<uintptr_t>(src) & 7) == 0;
}

// present = false: the plane does not exist (padding of a plane group);
// no row passes the window test, so nothing is loaded and the columns are zero.  (A branch
// around the call with a zero fill on the other side makes the compiler merge the stores
// of both sides into stores through a selected address, which parks the columns in
// scratch memory.)
// SPLIT (PAIRS = 0 only): the lane's columns are l and l + N/2 instead of 2l and 2l + 1, so
// that a load instruction reads neighbouring floats into neighbouring lanes; goes with
// columnPassForward<N, true>.
template <int N, int PAIRS = 2, bool SPLIT = false>
__device__ __forceinline__ void loadColumnsWindow(const float* src, int sy, int sx, int hWindow,
                                                  int w, int padL, int padU, int l,
                                                  c32 (&z0)[N / 2], c32 (&z1)[N / 2],
                                                  bool present = true) {
  static_assert(!SPLIT || PAIRS == 0, "split columns are loaded one float at a time");
  if constexpr (PAIRS == 2) {
    if (windowMovesAsPairs(src, sy, sx, w, padL))
      loadColumnsWindow<N, 1>(src, sy, sx, hWindow, w, padL, padU, l, z0, z1, present);
    else
      loadColumnsWindow<N, 0>(src, sy, sx, hWindow, w, padL, padU, l, z0, z1, present);
    return;
  }
  const int xa = (SPLIT ? l : 2 * l) - padL, xb = xa + (SPLIT ? N / 2 : 1);
  const bool va = (unsigned)xa < (unsigned)w, vb = (unsigned)xb < (unsigned)w;
  const int h = present ? hWindow : 0;  // rows that pass the window test
  const int yEnd = padU + h;
  // rows in batches of 8: a batch that lies wholly below the window (the same for
  // every lane) issues no loads - a 5 x 5 filter plane costs 16 loads, not 2N
  if constexpr (PAIRS == 1) {
    const float* pp = src + min(max(xa, 0), w - 2);
    // (zeroed up front rather than in an else branch: with stores to the same elements
    // on both sides of a branch the compiler merges them into stores through a selected
    // address, and the elements then live in scratch memory)
    float2 r[N];
    staticFor<N>([&](auto yy) { r[decltype(yy)::value] = float2{0.0f, 0.0f}; });
    staticFor<(N + 7) / 8>([&](auto bb) {
      constexpr int y0 = 8 * decltype(bb)::value;
      constexpr int y1 = y0 + 8 < N ? y0 + 8 : N;
      if (y0 < yEnd) {
        staticFor<y1 - y0>([&](auto yy) {
          constexpr int y = y0 + decltype(yy)::value;
          r[y] = *reinterpret_cast<const float2*>(pp + (long)min(max(y - padU, 0), hWindow - 1) * sy);
        });
      }
    });
    staticFor<N / 2>([&](auto jj) {
      constexpr int j = decltype(jj)::value;
      const bool v0 = va && (unsigned)(2 * j - padU) < (unsigned)h;
      const bool v1 = va && (unsigned)(2 * j + 1 - padU) < (unsigned)h;
      z0[j] = c32{v0 ? r[2 * j].x : 0.0f, v1 ? r[2 * j + 1].x : 0.0f};
      z1[j] = c32{v0 ? r[2 * j].y : 0.0f, v1 ? r[2 * j + 1].y : 0.0f};
    });
  } else {
    const float* pa = src + (long)min(max(xa, 0), w - 1) * sx;
    const float* pb = src + (long)min(max(xb, 0), w - 1) * sx;
    float ra[N], rb[N];
    staticFor<N>([&](auto yy) { ra[decltype(yy)::value] = rb[decltype(yy)::value] = 0.0f; });
    staticFor<(N + 7) / 8>([&](auto bb) {
      constexpr int y0 = 8 * decltype(bb)::value;
      constexpr int y1 = y0 + 8 < N ? y0 + 8 : N;
      if (y0 < yEnd) {
        staticFor<y1 - y0>([&](auto yy) {
          constexpr int y = y0 + decltype(yy)::value;
          const long oy = (long)min(max(y - padU, 0), hWindow - 1) * sy;
          ra[y] = pa[oy];
          rb[y] = pb[oy];
        });
      }
    });
    staticFor<N / 2>([&](auto jj) {
      constexpr int j = decltype(jj)::value;
      const bool v0 = (unsigned)(2 * j - padU) < (unsigned)h, v1 = (unsigned)(2 * j + 1 - padU) < (unsigned)h;
      z0[j] = c32{v0 && va ? ra[2 * j] : 0.0f, v1 && va ? ra[2 * j + 1] : 0.0f};
      z1[j] = c32{v0 && vb ? rb[2 * j] : 0.0f, v1 && vb ? rb[2 * j + 1] : 0.0f};
    });
  }
}

// The same two columns for callers whose window geometry differs from lane to
// lane of a wave (tile descriptors of different planes): the per-row terms are
// then vector arithmetic, and skipping the loads outside the window (tiles with
// 9 x 9 filters load 81 of 1024 samples) costs less than clamping every address.
template <int N>
__device__ __forceinline__ void loadColumnsWindowPerLane(const float* src, int sy, int sx, int h,
                                                         int w, int padL, int padU, int l,
                                                         c32 (&z0)[N / 2], c32 (&z1)[N / 2]) {
  const int xa = 2 * l - padL, xb = xa + 1;
  const bool va = (unsigned)xa < (unsigned)w, vb = (unsigned)xb < (unsigned)w;
  // element (y, xa) of the plane is pa[y * sy]; pa itself may point outside the
  // window and is only dereferenced under the tests
  // (global address space stated explicitly: the plane pointer comes out of a
  // descriptor in memory, and a generic pointer would make these flat loads)
  typedef const __attribute__((address_space(1))) float* GlobalPtr;
  // When every lane of the wave sees rows that start on 8-byte boundaries and a
  // window whose left edge and width are even, its two columns are one 8-byte word
  // per row, inside or outside the window together.
  const bool pairs = sx == 1 && ((sy | padL | w) & 1) == 0 &&
                     (reinterpret_cast<uintptr_t>(src) & 7) == 0;
  if (__builtin_amdgcn_ballot_w64(!pairs) == 0) {
    typedef float Pair __attribute__((ext_vector_type(2)));
    typedef const __attribute__((address_space(1))) Pair* GlobalPtr2;
    GlobalPtr2 pp = (GlobalPtr2)(src + xa - (long)padU * sy);
    const int sy2 = sy / 2;
    Pair r[N];
    // ... and when every lane's window covers the whole transform (the inner tiles of a
    // larger image), nothing is zeroed and nothing is tested row by row
    const bool whole = padU == 0 && padL == 0 && h >= N && w >= N;
    if (__builtin_amdgcn_ballot_w64(!whole) == 0) {
      staticFor<N>([&](auto yy) {
        constexpr int y = decltype(yy)::value;
        r[y] = pp[(long)y * sy2];
      });
      staticFor<N / 2>([&](auto jj) {
        constexpr int j = decltype(jj)::value;
        z0[j] = c32{r[2 * j].x, r[2 * j + 1].x};
        z1[j] = c32{r[2 * j].y, r[2 * j + 1].y};
      });
      return;
    }
    staticFor<N>([&](auto yy) {
      constexpr int y = decltype(yy)::value;
      r[y] = Pair{0.0f, 0.0f};
      if ((unsigned)(y - padU) < (unsigned)h && va) r[y] = pp[(long)y * sy2];
    });
    staticFor<N / 2>([&](auto jj) {
      constexpr int j = decltype(jj)::value;
      z0[j] = c32{r[2 * j].x, r[2 * j + 1].x};
      z1[j] = c32{r[2 * j].y, r[2 * j + 1].y};
    });
    return;
  }
  GlobalPtr pa = (GlobalPtr)(src + (long)xa * sx - (long)padU * sy);
  GlobalPtr pb = pa + sx;
  float ra[N], rb[N];
  staticFor<N>([&](auto yy) {
    constexpr int y = decltype(yy)::value;
    const bool vy = (unsigned)(y - padU) < (unsigned)h;
    ra[y] = 0.0f;
    rb[y] = 0.0f;
    if (vy && va) ra[y] = pa[(long)y * sy];
    if (vy && vb) rb[y] = pb[(long)y * sy];
  });
  staticFor<N / 2>([&](auto jj) {
    constexpr int j = decltype(jj)::value;
    z0[j] = c32{ra[2 * j], ra[2 * j + 1]};
    z1[j] = c32{rb[2 * j], rb[2 * j + 1]};
  });
}

// Column pass (forward): N/2-point FFTs of the two packed columns, real-input
// fix-up, packed rows written to the plane buffer.
template <int N, bool SPLIT = false>
__device__ __forceinline__ void columnPassForward(c32 (&z0)[N / 2], c32 (&z1)[N / 2], c32* plane,
                                                  int l) {
  constexpr int H = N / 2, RS = PlaneCfg<N>::RS;
  regFFT<H, true>(z0);
  regFFT<H, true>(z1);
  c32 p0[H], p1[H];
  realFixupForward<H>(z0, p0);
  realFixupForward<H>(z1, p1);
  if constexpr (SPLIT) {  // columns l and l + N/2
    c32* dst = plane + l;
    staticFor<H>([&](auto rr) {
      constexpr int r = decltype(rr)::value;
      dst[r * RS] = p0[r];
      dst[r * RS + H] = p1[r];
    });
  } else {
    c32* dst = plane + 2 * l;
    staticFor<H>([&](auto rr) {
      constexpr int r = decltype(rr)::value;
      ldsStore4(dst + r * RS, p0[r], p1[r]);
    });
  }
}

// Row pass: lane l transforms packed row l in place (natural order in and out).
template <int N, bool FWD>
__device__ __forceinline__ void rowPassInPlace(c32* plane, int l) {
  constexpr int RS = PlaneCfg<N>::RS;
  c32 row[N];
  c32* p = plane + l * RS;
  staticFor<N / 2>([&](auto jj) {
    constexpr int j = decltype(jj)::value;
    float4 v = ldsLoad4(p + 2 * j);
    row[2 * j] = c32{v.x, v.y};
    row[2 * j + 1] = c32{v.z, v.w};
  });
  regFFT<N, FWD>(row);
  staticFor<N / 2>([&](auto jj) {
    constexpr int j = decltype(jj)::value;
    ldsStore4(p + 2 * j, row[slot<N>(2 * j)], row[slot<N>(2 * j + 1)]);
  });
}

// Column pass (inverse): reads packed rows of columns 2l, 2l+1, undoes the
// real-input fix-up and runs the inverse N/2-point FFTs.  On return
// z[slot<N/2>(j)] = (X[2j][x], X[2j+1][x]) * N*N for the two columns.
// SPLIT: the lane takes columns l and l + N/2 instead of 2l and 2l + 1 (two 8-byte LDS
// reads per row instead of one 16-byte read), so that a store instruction of
// storeColumnsWindow<..., SPLIT> writes neighbouring floats from neighbouring lanes.
template <int N, bool SPLIT = false>
__device__ __forceinline__ void columnPassInverse(const c32* plane, int l, c32 (&z0)[N / 2],
                                                  c32 (&z1)[N / 2]) {
  constexpr int H = N / 2, RS = PlaneCfg<N>::RS;
  c32 p0[H], p1[H];
  if constexpr (SPLIT) {
    const c32* src = plane + l;
    staticFor<H>([&](auto rr) {
      constexpr int r = decltype(rr)::value;
      p0[r] = src[r * RS];
      p1[r] = src[r * RS + H];
    });
  } else {
    const c32* src = plane + 2 * l;
    staticFor<H>([&](auto rr) {
      constexpr int r = decltype(rr)::value;
      float4 v = ldsLoad4(src + r * RS);
      p0[r] = c32{v.x, v.y};
      p1[r] = c32{v.z, v.w};
    });
  }
  realFixupInverse<H>(p0, z0);
  realFixupInverse<H>(p1, z1);
  regFFT<H, false>(z0);
  regFFT<H, false>(z1);
}

// Two columns of results through a bounds-checked strided view (crop on store).
// ACC adds the scaled result to what the view holds instead of replacing it;
// ATOMIC does that with an atomic add (several workgroups contribute to one view).
// PAIRS: the caller guarantees windowMovesAsPairs() for the view, so the lane's two
// columns of a row are one 8-byte word, inside or outside the window together.
// SPLIT: z0 / z1 are columns l and l + N/2 (columnPassInverse<N, true>): each of a row's
// two store instructions then writes a contiguous run per plane instead of every other
// float.
template <int N, bool ACC = false, bool ATOMIC = false, bool PAIRS = false, bool SPLIT = false>
__device__ __forceinline__ void storeColumnsWindow(float* dst, int sy, int sx, int h, int w, int padL,
                                                   int padU, int l, const c32 (&z0)[N / 2],
                                                   const c32 (&z1)[N / 2], float scale) {
  static_assert(!(PAIRS && SPLIT), "paired stores need neighbouring columns in one lane");
  // The column tests are per lane and the same for every row; the row test is
  // wave-uniform (a scalar branch).  The two columns of a row are stored back to
  // back so that both halves of a cache line reach L2 together.
  const int xa = (SPLIT ? l : 2 * l) - padL, xb = xa + (SPLIT ? N / 2 : 1);
  const bool va = (unsigned)xa < (unsigned)w, vb = (unsigned)xb < (unsigned)w;
  if constexpr (PAIRS) {
    static_assert(!ATOMIC, "paired stores replace or add in place");
    float2* pp = reinterpret_cast<float2*>(dst + xa);
    const int sy2 = sy / 2;
    staticFor<N>([&](auto yy) {
      constexpr int y = decltype(yy)::value;
      if ((unsigned)(y - padU) < (unsigned)h) {
        const c32 a = z0[slot<N / 2>(y / 2)], c = z1[slot<N / 2>(y / 2)];
        float2 v = float2{(y % 2 ? a.y : a.x) * scale, (y % 2 ? c.y : c.x) * scale};
        float2* q = pp + (long)(y - padU) * sy2;
        if (va) {
          if constexpr (ACC) {
            const float2 o = *q;
            v.x += o.x;
            v.y += o.y;
          }
          // (whole 8-byte words leave with the nontemporal hint: 281 -> 271 us for the
          // forward pass of a 16 x 32 x 256 x 256 layer; on the 4-byte stores of odd
          // widths below the hint costs 6 %, partly written lines no longer meet in L2)
          if constexpr (ACC)
            *q = v;
          else
            streamStore(q, v);
        }
      }
    });
    return;
  }
  // (the view is device memory; said explicitly because a pointer that comes out of a
  // descriptor in memory is generic and would make these flat instructions)
  typedef __attribute__((address_space(1))) float* GlobalPtr;
  GlobalPtr pa = (GlobalPtr)(dst + (long)xa * sx);
  GlobalPtr pb = (GlobalPtr)(dst + (long)xb * sx);
  auto put = [&](GlobalPtr q, float r) __attribute__((always_inline)) {
    if constexpr (ATOMIC)
      atomicAdd((float*)q, r * scale);
    else if constexpr (ACC)
      *q += r * scale;
    else
      *q = r * scale;
  };
  staticFor<N>([&](auto yy) {
    constexpr int y = decltype(yy)::value;
    if ((unsigned)(y - padU) < (unsigned)h) {
      const long oy = (long)(y - padU) * sy;
      const c32 a = z0[slot<N / 2>(y / 2)], c = z1[slot<N / 2>(y / 2)];
      if (va) put(pa + oy, y % 2 ? a.y : a.x);
      if (vb) put(pb + oy, y % 2 ? c.y : c.x);
    }
  });
}

}  // namespace fbfft_amd
