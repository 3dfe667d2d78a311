// TEST INFRASTRUCTURE ONLY.  This file is the CPU restatement ("oracle") of the
// reference's fbfft path.  Only the test-suite, the smoke check and the
// benchmark's cpu_baseline leg may load it; no product code path links or calls
// anything in this directory.
//
// Two families of functions live here:
//
//  * orc_*   - a host transcription of the reference's fp32 algorithm: the same
//              radix-2 decimation-in-frequency butterflies, the same
//              correctly-rounded 128-entry twiddle table, the same real-input
//              packing tricks and the same operand layouts, with GPU lanes
//              restated as array indices.  Compiled with -ffp-contract=off so
//              that a complex product is exactly (ac - bd, ad + bc) as in
//              cuCmulf (Complex.cuh:69-71).
//  * ref64_* - definitions in double precision: naive DFT sums and direct
//              valid cross-correlation.  These follow no reference file; they
//              are what the mathematics fixes and are used to pin the orc_*
//              functions and the GPU kernels alike.
//
// Parity status: the reference ships no test, golden vector or fixture for this
// path and cannot be compiled here (CUDA only), so "parity unpinned by the
// reference's own tests" applies to every orc_* function.  Each one is pinned
// instead by ref64_* (itself pinned by closed forms and numpy.fft in
// tests/test_oracle.py).  Two reference quirks are pinned by the transcription
// alone: the 1D padL store asymmetry (FBFFTCommon.cuh:425-427) and the lane-0
// treatment of non-Hermitian input in the 2D inverse (FFT2D32.cuh:310-316).
//
// Multiplications by the twiddle table's (1, +-0) entry, which the reference
// performs on the "lower" lanes of every warp butterfly
// (FBFFTCommon.cuh:460-468), are exact identities on finite data and are elided.

#include <cmath>
#include <cstdint>
#include <cstring>
#include <vector>

#ifdef _OPENMP
#include <omp.h>
#endif

namespace {

struct cf {
  float re, im;
};

inline cf mk(float re, float im = 0.0f) { return cf{re, im}; }
inline cf operator+(cf a, cf b) { return cf{a.re + b.re, a.im + b.im}; }
inline cf operator-(cf a, cf b) { return cf{a.re - b.re, a.im - b.im}; }
inline cf operator-(cf a) { return cf{-a.re, -a.im}; }
// cuCmulf ordering (Complex.cuh:69-71)
inline cf operator*(cf a, cf b) {
  return cf{a.re * b.re - a.im * b.im, a.re * b.im + a.im * b.re};
}
inline cf conj(cf a) { return cf{a.re, -a.im}; }
// Complex::transpose swaps the real and imaginary parts (Complex.cuh:98-101)
inline cf swp(cf a) { return cf{a.im, a.re}; }

const uint32_t kTwiddleBits[256] = {
#include "twiddles_f32.inc"
};

// entry idx of the table: e^{+i*pi*idx/128}  (Twiddles.cuh:322-453)
inline cf tableEntry(int idx) {
  cf r;
  std::memcpy(&r.re, &kTwiddleBits[2 * idx], 4);
  std::memcpy(&r.im, &kTwiddleBits[2 * idx + 1], 4);
  return r;
}

// W_M^k in the direction of the transform: the reference fetches entry
// 2*k*(128/M) and conjugates it for the forward FFT (FBFFTCommon.cuh:124-136);
// cexp<M>(2k) in the unrolled register FFTs is the same entry
// (Twiddles.cuh:254-306).
//
// Deviation: for M = 256 the reference's integer expression 2*k*(128/256)
// truncates to entry 0 for every k, so its 256-point 1D transform multiplies by
// 1 throughout and does not compute a DFT.  The oracle (and the product) use
// the entry the formula means, k*256/M, which is identical for every M <= 128.
inline cf root(int M, int k, bool forward) {
  cf w = tableEntry(k * 256 / M);
  return forward ? conj(w) : w;
}

// cexp<H>(i) = e^{+i*pi*i/H}, H <= 64 (Twiddles.cuh:254-306 for H <= 32)
inline cf cexpHalf(int H, int i) { return tableEntry(i * (128 / H)); }

inline int log2i(int n) {
  int l = 0;
  while ((1 << l) < n) ++l;
  return l;
}

inline int bitrev(int x, int bits) {
  int r = 0;
  for (int i = 0; i < bits; ++i) r |= ((x >> i) & 1) << (bits - 1 - i);
  return r;
}

inline bool isPow2(int n) { return n > 0 && (n & (n - 1)) == 0; }

// Radix-2 decimation in frequency over v[0..N) with stride, in place; result is
// left in bit-reversed order.  One restatement serves the warp butterfly
// (FBFFTCommon.cuh:432-474 and the register-twiddle variant :476-495), the
// cross-register stages for N > 32 (:616-708; their rebalanced twiddles are
// plain table entries) and the unrolled FFT4/8/16/32 (FFT2D32.cuh:132-219).  In
// all of them the sum / difference is formed first and the difference is then
// multiplied by the twiddle W_M^k; W_M^0 is the table's (1, +-0) entry.
void difStages(cf* v, int stride, int N, bool forward) {
  for (int M = N; M >= 2; M >>= 1) {
    const int half = M / 2;
    for (int base = 0; base < N; base += M) {
      for (int k = 0; k < half; ++k) {
        cf& lo = v[(base + k) * stride];
        cf& hi = v[(base + k + half) * stride];
        cf s = lo + hi;
        cf d = lo - hi;
        if (k > 0) d = d * root(M, k, forward);
        lo = s;
        hi = d;
      }
    }
  }
}

void bitReverse(cf* v, int stride, int N) {
  const int bits = log2i(N);
  for (int i = 0; i < N; ++i) {
    int j = bitrev(i, bits);
    if (i < j) {
      cf t = v[i * stride];
      v[i * stride] = v[j * stride];
      v[j * stride] = t;
    }
  }
}

// ---------------------------------------------------------------------------
// 1D R2C / C2R  (FBFFTCommon.cuh:307-351 load1DR2C, :387-430 store1DR2C,
// :710-794 kernel bodies, FBFFT-inl.cuh:19-150 dispatch)
// ---------------------------------------------------------------------------

bool supported1D(int N) { return isPow2(N) && N >= 2 && N <= 256; }

void fbfft1dPair(const float* real, int B, int N, int padL, float* cplx, int b) {
  const int nc = N / 2 + 1;
  const bool second = (b + 1 < B);
  std::vector<cf> v(N);
  for (int x = 0; x < N; ++x) {
    // the reference tests "0 <= x - padL && x < size": a right shift that drops
    // the last padL samples (FBFFTCommon.cuh:325)
    if (0 <= x - padL && x < N) {
      v[x] = mk(real[(size_t)b * N + x - padL],
                second ? real[(size_t)(b + 1) * N + x - padL] : 0.0f);
    } else {
      v[x] = mk(0.0f);
    }
  }
  difStages(v.data(), 1, N, true);
  bitReverse(v.data(), 1, N);
  for (int x = 0; x < nc; ++x) {
    cf me = v[x];
    cf other = v[(N - x) % N];
    float* o1 = cplx + ((size_t)b * nc + x) * 2;
    o1[0] = 0.5f * (me.re + other.re);
    o1[1] = 0.5f * (me.im - other.im);
    if (second) {
      float* o2 = cplx + ((size_t)(b + 1) * nc + x) * 2;
      o2[0] = 0.5f * (me.im + other.im);
      o2[1] = 0.5f * (-me.re + other.re);
    }
  }
}

void fbifft1dPair(const float* cplx, int B, int N, int padL, float* real, int b) {
  const int nc = N / 2 + 1;
  const bool second = (b + 1 < B);
  std::vector<cf> v(N);
  auto fetch = [&](int row, int x) {
    const float* p = cplx + (size_t)row * nc * 2;
    if (x < nc) return mk(p[2 * x], p[2 * x + 1]);
    int m = 2 * (nc - 1) - x;
    return conj(mk(p[2 * m], p[2 * m + 1]));
  };
  for (int x = 0; x < N; ++x) {
    cf t1 = fetch(b, x);
    cf t2 = second ? fetch(b + 1, x) : mk(0.0f);
    v[x] = mk(t1.re - t2.im, t1.im + t2.re);
  }
  difStages(v.data(), 1, N, false);
  bitReverse(v.data(), 1, N);
  for (int x = 0; x < N; ++x) {
    if (0 <= x - padL && x - padL < N) {
      // row b is written at x, row b+1 at x - padL (FBFFTCommon.cuh:425-427)
      real[(size_t)b * N + x] = v[x].re;
      if (second) real[(size_t)(b + 1) * N + x - padL] = v[x].im;
    }
  }
}

// ---------------------------------------------------------------------------
// 2D, N in {8, 16, 32}  (FFT2D32.cuh)
// Working set of one plane: a[i][x], i = 0..N/2-1 "registers", x = 0..N-1 lanes.
// ---------------------------------------------------------------------------

inline bool inBounds2(int y, int x, int padU, int padL, int h, int w) {
  // MemoryAccess.cuh:19-25
  return (unsigned)(y - padU) < (unsigned)h && (unsigned)(x - padL) < (unsigned)w;
}

// fbfft2DVerticalCoreForward (FFT2D32.cuh:257-299)
void coreForward(cf* a, int N) {
  const int H = N / 2;
  for (int x = 0; x < N; ++x) {
    cf* col = a + x;  // stride N between registers
    difStages(col, N, H, true);
    bitReverse(col, N, H);
    col[0] = conj(col[0]) + swp(col[0]);
    for (int i = 1; i < H / 2; ++i) {
      cf ai = col[i * N], aj = col[(H - i) * N];
      cf Si = mk(0.5f) * (ai + conj(aj));
      cf Di = mk(0.5f) * (ai - conj(aj));
      col[i * N] = Si - Di * swp(cexpHalf(H, i));
      col[(H - i) * N] = conj(Si) - (-conj(Di)) * swp(cexpHalf(H, H - i));
    }
    col[(H / 2) * N] = conj(col[(H / 2) * N]);
  }
  for (int i = 0; i < H; ++i) {
    difStages(a + i * N, 1, N, true);
    bitReverse(a + i * N, 1, N);
  }
}

// fbfft2DVerticalCoreInverse (FFT2D32.cuh:302-358).  When !packedInput the
// caller supplies a[N/2] as well.
void coreInverse(cf* a, int N, bool packedInput) {
  const int H = N / 2;
  if (!packedInput) {
    for (int x = 0; x < N; ++x) {
      if (x > 0) {
        a[x] = a[x] - conj(swp(a[H * N + x]));
      } else {
        a[x] = mk(a[x].re, a[H * N + x].re);
      }
    }
  }
  for (int i = 0; i < H; ++i) {
    difStages(a + i * N, 1, N, false);
    bitReverse(a + i * N, 1, N);
  }
  for (int x = 0; x < N; ++x) {
    cf* col = a + x;
    col[0] = conj(col[0]) + swp(col[0]);
    for (int i = 1; i < H / 2; ++i) {
      cf ai = col[i * N], aj = col[(H - i) * N];
      cf Si = ai + conj(aj);
      cf Di = ai - conj(aj);
      col[i * N] = Si - Di * conj(swp(cexpHalf(H, i)));
      col[(H - i) * N] = conj(Si) - ((-conj(Di)) * conj(swp(cexpHalf(H, H - i))));
    }
    {
      cf am = col[(H / 2) * N];
      cf Si = am + conj(am);
      cf Di = am - conj(am);
      col[(H / 2) * N] = Si - ((-conj(Di)) * conj(swp(cexpHalf(H, H / 2))));
    }
    difStages(col, N, H, false);
    bitReverse(col, N, H);
  }
}

void loadPacked(cf* a, int N, const float* plane, int h, int w, int rowStride,
                int padL, int padU) {
  // FFT2D32.cuh:387-393
  for (int i = 0; i < N; i += 2) {
    for (int x = 0; x < N; ++x) {
      float f1 = inBounds2(i, x, padU, padL, h, w)
                     ? plane[(size_t)(i - padU) * rowStride + x - padL] : 0.0f;
      float f2 = inBounds2(i + 1, x, padU, padL, h, w)
                     ? plane[(size_t)(i + 1 - padU) * rowStride + x - padL] : 0.0f;
      a[(i / 2) * N + x] = mk(f1, f2);
    }
  }
}

// Unpack rows 0 and N/2 of the packed forward result (FFT2D32.cuh:403-420)
inline void unpackRow0(const cf* a, int N, int x, cf* r0, cf* rN2) {
  if (x > 0) {
    cf other = a[N - x];
    *r0 = mk(0.5f) * (conj(other) + a[x]);
    *rN2 = mk(0.5f) * swp(conj(conj(other) - a[x]));
  } else {
    *r0 = mk(a[0].re);
    *rN2 = mk(a[0].im);
  }
}

// packed: the Unpack = false store (FFT2D32.cuh:421-427), out is [N/2][N]
void fbfft2dSmallPlane(const float* plane, int h, int w, int N, int padL, int padU,
                       float* out, bool packed = false) {
  const int H = N / 2;
  std::vector<cf> a((size_t)H * N);
  loadPacked(a.data(), N, plane, h, w, w, padL, padU);
  coreForward(a.data(), N);
  cf* o = reinterpret_cast<cf*>(out);  // [N/2+1][N]
  if (packed) {
    for (int i = 0; i < H; ++i)
      for (int x = 0; x < N; ++x) o[i * N + x] = a[i * N + x];
    return;
  }
  for (int i = 1; i < H; ++i)
    for (int x = 0; x < N; ++x) o[i * N + x] = a[i * N + x];
  for (int x = 0; x < N; ++x) unpackRow0(a.data(), N, x, &o[x], &o[H * N + x]);
}

// packed: PackedInput = true (FFT2D32.cuh:446-458), in is [N/2][N]
void fbifft2dSmallPlane(const float* in, int N, int h, int w, int padL, int padU,
                        float* plane, bool packed = false) {
  const int H = N / 2;
  std::vector<cf> a((size_t)(H + 1) * N);
  std::memcpy(a.data(), in, sizeof(cf) * (size_t)(packed ? H : H + 1) * N);
  coreInverse(a.data(), N, packed);
  // FFT2D32.cuh:462-469
  for (int i = 0; i < N; i += 2) {
    for (int x = 0; x < N; ++x) {
      if (inBounds2(i, x, padU, padL, h, w))
        plane[(size_t)(i - padU) * w + x - padL] = a[(i / 2) * N + x].re;
      if (inBounds2(i + 1, x, padU, padL, h, w))
        plane[(size_t)(i + 1 - padU) * w + x - padL] = a[(i / 2) * N + x].im;
    }
  }
}

// ---------------------------------------------------------------------------
// 2D, N in {64, 128}: two passes through a scratch buffer.
// Forward  (FBFFT2D-inl.cuh:230-317 pass 1, :321-418 pass 2)
// Inverse  (FBIFFT2D-inl.cuh:61-138 loads, :252-356 pass 1, :360-474 pass 2)
// ---------------------------------------------------------------------------

void fbfft2dLargePlane(const float* plane, int h, int w, int N, int padL, int padU,
                       float* out) {
  const int nc = N / 2 + 1;
  std::vector<cf> scratch((size_t)N * nc);  // [y][kx]
  std::vector<cf> v(N);
  for (int y = 0; y < N; ++y) {
    for (int x = 0; x < N; ++x)
      v[x] = mk(inBounds2(y, x, padU, padL, h, w)
                    ? plane[(size_t)(y - padU) * w + x - padL] : 0.0f, 0.0f);
    difStages(v.data(), 1, N, true);
    bitReverse(v.data(), 1, N);
    for (int x = 0; x < nc; ++x) scratch[(size_t)y * nc + x] = v[x];
  }
  cf* o = reinterpret_cast<cf*>(out);  // [kx][ky]
  for (int kx = 0; kx < nc; ++kx) {
    for (int y = 0; y < N; ++y) v[y] = scratch[(size_t)y * nc + kx];
    difStages(v.data(), 1, N, true);
    bitReverse(v.data(), 1, N);
    for (int ky = 0; ky < N; ++ky) o[(size_t)kx * N + ky] = v[ky];
  }
}

// Planes b0 and b1 (b1 < 0: absent) are carried as the real and imaginary part
// of one complex inverse transform (FBIFFT2D-inl.cuh:293-296, :465-469).
void fbifft2dLargePair(const float* in0, const float* in1, int N, int h, int w,
                       int padL, int padU, float* plane0, float* plane1) {
  const int nc = N / 2 + 1;
  std::vector<cf> scratch((size_t)N * N);  // [row][col]
  std::vector<cf> v(N);
  auto expand = [&](const float* in, int row, int col) {
    const cf* p = reinterpret_cast<const cf*>(in);
    if (row < nc) return p[(size_t)row * N + col];
    int rrow = N - row, ccol = (N - col) % N;
    return conj(p[(size_t)rrow * N + ccol]);
  };
  for (int row = 0; row < N; ++row) {
    for (int col = 0; col < N; ++col) {
      cf c = expand(in0, row, col);
      if (in1) {
        cf t = expand(in1, row, col);
        c = c + mk(-t.im, t.re);
      }
      v[col] = c;
    }
    difStages(v.data(), 1, N, false);
    bitReverse(v.data(), 1, N);
    for (int col = 0; col < N; ++col) scratch[(size_t)row * N + col] = v[col];
  }
  for (int x = 0; x < N; ++x) {  // x: second index of the scratch, output row
    for (int y = 0; y < N; ++y) v[y] = scratch[(size_t)y * N + x];
    difStages(v.data(), 1, N, false);
    bitReverse(v.data(), 1, N);
    for (int ccol = 0; ccol < N; ++ccol) {
      if (inBounds2(x, ccol, padU, padL, h, w)) {
        plane0[(size_t)(x - padU) * w + ccol - padL] = v[ccol].re;
        if (plane1) plane1[(size_t)(x - padU) * w + ccol - padL] = v[ccol].im;
      }
    }
  }
}

// ---------------------------------------------------------------------------
// 2D, N in {2, 4}: the warp kernel that the entry point falls through to for
// sizes the register kernels do not cover (FBFFT2D-inl.cuh:124-222, dispatch
// :571-615).  Planes b and b+1 ride as the real and imaginary part of one
// complex row transform (load2DR2C, :45-69), the two spectra are separated with
// the Hermitian split (:171-183), transposed, and the first N/2+1 columns are
// transformed again; store2D (:71-85) writes cplx[b][kx][ky], the same layout as
// N >= 64.  The inverse for these sizes (FBIFFT2D-inl.cuh:188-247, dispatch
// :684-712) is the one-kernel form of fbifft2dLargePair above with the same
// plane pairing b, b + ceil(B/2).
// ---------------------------------------------------------------------------

void fbfft2dWarpPair(const float* p0, const float* p1, int h, int w, int N, int padL, int padU,
                     float* out0, float* out1) {
  const int nc = N / 2 + 1;
  std::vector<cf> A((size_t)N * N), Bv((size_t)N * N), v(N);  // [y][kx]
  for (int y = 0; y < N; ++y) {
    for (int x = 0; x < N; ++x) {
      if (inBounds2(y, x, padU, padL, h, w)) {
        const size_t i = (size_t)(y - padU) * w + x - padL;
        v[x] = mk(p0[i], p1 ? p1[i] : 0.0f);
      } else {
        v[x] = mk(0.0f, 0.0f);
      }
    }
    difStages(v.data(), 1, N, true);
    bitReverse(v.data(), 1, N);
    for (int x = 0; x < N; ++x) {
      const cf me = v[x], other = v[(N - x) % N];
      A[(size_t)y * N + x] = mk(0.5f * (me.re + other.re), 0.5f * (me.im - other.im));
      Bv[(size_t)y * N + x] = mk(0.5f * (me.im + other.im), 0.5f * (-me.re + other.re));
    }
  }
  for (int which = 0; which < 2; ++which) {
    float* out = which == 0 ? out0 : out1;
    if (!out) continue;
    const std::vector<cf>& src = which == 0 ? A : Bv;
    cf* o = reinterpret_cast<cf*>(out);
    for (int kx = 0; kx < nc; ++kx) {
      for (int y = 0; y < N; ++y) v[y] = src[(size_t)y * N + kx];
      difStages(v.data(), 1, N, true);
      bitReverse(v.data(), 1, N);
      for (int ky = 0; ky < N; ++ky) o[(size_t)kx * N + ky] = v[ky];
    }
  }
}

// TiledDeviceTensor<float,4> (FFTIteratedConvolution.cuh:71-88) with the
// DeviceTensor member order data, stride, size (DeviceTensor.cuh:237-245).
struct TileDesc {
  int padL;
  int padU;
  float* data;
  int stride[4];
  int size[4];
};
static_assert(sizeof(TileDesc) == 48, "descriptor is 48 bytes");

inline float* at4(const TileDesc& t, int a, int b, int y, int x) {
  return t.data + (size_t)a * t.stride[0] + (size_t)b * t.stride[1] +
         (size_t)y * t.stride[2] + (size_t)x * t.stride[3];
}

void loadPackedTile(cf* a, int N, const TileDesc& t, int n, int c) {
  const int h = t.size[2], w = t.size[3];
  for (int i = 0; i < N; i += 2) {
    for (int x = 0; x < N; ++x) {
      float f1 = inBounds2(i, x, t.padU, t.padL, h, w)
                     ? *at4(t, n, c, i - t.padU, x - t.padL) : 0.0f;
      float f2 = inBounds2(i + 1, x, t.padU, t.padL, h, w)
                     ? *at4(t, n, c, i + 1 - t.padU, x - t.padL) : 0.0f;
      a[(i / 2) * N + x] = mk(f1, f2);
    }
  }
}

void storePackedTile(const cf* a, int N, const TileDesc& t, int n, int c, float scale) {
  const int h = t.size[2], w = t.size[3];
  for (int i = 0; i < N; i += 2) {
    for (int x = 0; x < N; ++x) {
      if (inBounds2(i, x, t.padU, t.padL, h, w))
        *at4(t, n, c, i - t.padU, x - t.padL) = a[(i / 2) * N + x].re * scale;
      if (inBounds2(i + 1, x, t.padU, t.padL, h, w))
        *at4(t, n, c, i + 1 - t.padU, x - t.padL) = a[(i / 2) * N + x].im * scale;
    }
  }
}

}  // namespace

extern "C" {

int orc_num_threads() {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

void orc_set_num_threads(int n) {
#ifdef _OPENMP
  omp_set_num_threads(n);
#else
  (void)n;
#endif
}

void orc_twiddle_table(float* out256) {
  std::memcpy(out256, kTwiddleBits, sizeof(kTwiddleBits));
}

// fbfft1D<1> (FBFFT-inl.cuh:19-87): real [B][N] -> cplx [B][N/2+1][2].
// Returns 0 (Success) or 1 (UnsupportedSize).
int orc_fbfft1d(const float* real, int B, int N, int padL, float* cplx) {
  if (!supported1D(N)) return 1;
#pragma omp parallel for schedule(static)
  for (int b = 0; b < B; b += 2) fbfft1dPair(real, B, N, padL, cplx, b);
  return 0;
}

// fbifft1D<1> (FBFFT-inl.cuh:89-150): cplx [B][N/2+1][2] -> real [B][N], gain N.
int orc_fbifft1d(const float* cplx, int B, int N, int padL, float* real) {
  if (!supported1D(N)) return 1;
#pragma omp parallel for schedule(static)
  for (int b = 0; b < B; b += 2) fbifft1dPair(cplx, B, N, padL, real, b);
  return 0;
}

// fbfft2D<1> (FBFFT2D-inl.cuh:450-669): real [B][h][w] (contiguous) placed at
// (padU, padL) of a zero N x N plane -> cplx [B][N/2+1][N][2].
// N in {8,16,32}: cplx[b][ky][kx]; N in {2,4} and N >= 64: cplx[b][kx][ky].
int orc_fbfft2d(const float* real, int B, int h, int w, int N, int padL, int padU,
                float* cplx) {
  if (!(N == 2 || N == 4 || N == 8 || N == 16 || N == 32 || N == 64 || N == 128)) return 1;
  const size_t inPlane = (size_t)h * w, outPlane = (size_t)(N / 2 + 1) * N * 2;
  if (N < 8) {
#pragma omp parallel for schedule(static)
    for (int b = 0; b < B; b += 2) {
      const bool two = b + 1 < B;
      fbfft2dWarpPair(real + b * inPlane, two ? real + (b + 1) * inPlane : nullptr, h, w, N, padL,
                      padU, cplx + b * outPlane, two ? cplx + (b + 1) * outPlane : nullptr);
    }
    return 0;
  }
#pragma omp parallel for schedule(static)
  for (int b = 0; b < B; ++b) {
    if (N <= 32)
      fbfft2dSmallPlane(real + b * inPlane, h, w, N, padL, padU, cplx + b * outPlane);
    else
      fbfft2dLargePlane(real + b * inPlane, h, w, N, padL, padU, cplx + b * outPlane);
  }
  return 0;
}

// fbifft2D<1> (FBIFFT2D-inl.cuh:529-742): cplx [B][N/2+1][N][2] ->
// real [B][h][w], gain N*N, cropped to the (padU, padL) window.
int orc_fbifft2d(const float* cplx, int B, int N, int h, int w, int padL, int padU,
                 float* real) {
  if (!(N == 2 || N == 4 || N == 8 || N == 16 || N == 32 || N == 64 || N == 128)) return 1;
  const size_t outPlane = (size_t)h * w, inPlane = (size_t)(N / 2 + 1) * N * 2;
  if (N >= 8 && N <= 32) {
#pragma omp parallel for schedule(static)
    for (int b = 0; b < B; ++b)
      fbifft2dSmallPlane(cplx + b * inPlane, N, h, w, padL, padU, real + b * outPlane);
  } else {
    const int half = (B + 1) / 2;  // gridDim.x of both inverse passes
#pragma omp parallel for schedule(static)
    for (int b = 0; b < half; ++b) {
      const int b1 = b + half;
      fbifft2dLargePair(cplx + b * inPlane, b1 < B ? cplx + b1 * inPlane : nullptr, N, h, w,
                        padL, padU, real + b * outPlane,
                        b1 < B ? real + b1 * outPlane : nullptr);
    }
  }
  return 0;
}

// fbfft2DVertical<..., Unpack = false> (FFT2D32.cuh:361-427): real [B][h][w] ->
// cplx [B][N/2][N][2], N in {8,16,32}; row 0 holds F[0][kx] + i F[N/2][kx].  The
// reference declares this store but instantiates no kernel with it
// (FFT2D32.cuh:473-502 use the default); the fused convolution kernels consume the
// same in-register form.
int orc_fbfft2d_packed(const float* real, int B, int h, int w, int N, int padL, int padU,
                       float* cplx) {
  if (!(N == 8 || N == 16 || N == 32)) return 1;
  const size_t inPlane = (size_t)h * w, outPlane = (size_t)(N / 2) * N * 2;
#pragma omp parallel for schedule(static)
  for (int b = 0; b < B; ++b)
    fbfft2dSmallPlane(real + b * inPlane, h, w, N, padL, padU, cplx + b * outPlane, true);
  return 0;
}

// fbifft2DVertical<..., PackedInput = true> (FFT2D32.cuh:430-470, core :302-358):
// cplx [B][N/2][N][2] -> real [B][h][w], gain N*N.
int orc_fbifft2d_packed(const float* cplx, int B, int N, int h, int w, int padL, int padU,
                        float* real) {
  if (!(N == 8 || N == 16 || N == 32)) return 1;
  const size_t outPlane = (size_t)h * w, inPlane = (size_t)(N / 2) * N * 2;
#pragma omp parallel for schedule(static)
  for (int b = 0; b < B; ++b)
    fbifft2dSmallPlane(cplx + b * inPlane, N, h, w, padL, padU, real + b * outPlane, true);
  return 0;
}

// The per-frequency contraction on packed spectra [..][..][N/2][N]: rows 1..N/2-1
// as orc_transpose_mm; row 0 by the product rule of the fused kernels
// (FFTIteratedConvolution.cuh:161-186 for a * conj(b), :317-337 for a * b, :483-504
// for the unpacking): with other = P[N - x], F0 = 0.5 (conj(other) + P),
// FH = 0.5 transpose(conj(conj(other) - P)), the rows multiply separately and
// acc += out0 + transpose(conj(outH)); lane 0 multiplies its two real pairs
// component by component.  op() conjugates the unpacked values.
void orc_transpose_mm_packed(const float* A, const float* B, float* C, int I, int J, int K, int N,
                             int conjA, int conjB, int accumulate, float invNorm) {
  const cf* a = reinterpret_cast<const cf*>(A);
  const cf* b = reinterpret_cast<const cf*>(B);
  cf* c = reinterpret_cast<cf*>(C);
  const int XY = N / 2 * N;
#pragma omp parallel for collapse(2) schedule(static)
  for (int i = 0; i < I; ++i) {
    for (int j = 0; j < J; ++j) {
      for (int xy = 0; xy < XY; ++xy) {
        cf acc = accumulate ? c[((size_t)i * J + j) * XY + xy] : mk(0.0f);
        for (int k = 0; k < K; ++k) {
          const cf* ap = conjA ? a + ((size_t)k * I + i) * XY : a + ((size_t)i * K + k) * XY;
          const cf* bp = conjB ? b + ((size_t)j * K + k) * XY : b + ((size_t)k * J + j) * XY;
          cf av = ap[xy], bv = bp[xy];
          if (xy >= N) {
            if (conjA) av = conj(av);
            if (conjB) bv = conj(bv);
            acc = av * bv + acc;
          } else if (xy > 0) {
            cf oa = ap[N - xy], ob = bp[N - xy];
            cf a0 = mk(0.5f) * (conj(oa) + av);
            cf aH = mk(0.5f) * swp(conj(conj(oa) - av));
            cf b0 = mk(0.5f) * (conj(ob) + bv);
            cf bH = mk(0.5f) * swp(conj(conj(ob) - bv));
            if (conjA) { a0 = conj(a0); aH = conj(aH); }
            if (conjB) { b0 = conj(b0); bH = conj(bH); }
            cf out0 = a0 * b0;
            cf outH = aH * bH;
            acc = acc + (out0 + swp(conj(outH)));
          } else {
            acc = acc + mk(av.re * bv.re, av.im * bv.im);
          }
        }
        acc.re *= invNorm;
        acc.im *= invNorm;
        c[((size_t)i * J + j) * XY + xy] = acc;
      }
    }
  }
}

// transposeMM (MM-inl.cuh:188-196 semantics, :302-326 accumulation order and
// scaling).  Operands are complex, xy innermost:
//   !conjA: A[I][K][XY]   conjA: A[K][I][XY]
//   !conjB: B[K][J][XY]   conjB: B[J][K][XY]
//   C[I][J][XY] = invNorm * ((accumulate ? C : 0) + sum_k opA * opB)
// Note that invNorm also scales the accumulated-into value (:322-324).
void orc_transpose_mm(const float* A, const float* B, float* C, int I, int J, int K, int XY,
                      int conjA, int conjB, int accumulate, float invNorm) {
  const cf* a = reinterpret_cast<const cf*>(A);
  const cf* b = reinterpret_cast<const cf*>(B);
  cf* c = reinterpret_cast<cf*>(C);
#pragma omp parallel for collapse(2) schedule(static)
  for (int i = 0; i < I; ++i) {
    for (int j = 0; j < J; ++j) {
      for (int xy = 0; xy < XY; ++xy) {
        cf acc = accumulate ? c[((size_t)i * J + j) * XY + xy] : mk(0.0f);
        for (int k = 0; k < K; ++k) {
          cf av = conjA ? a[((size_t)k * I + i) * XY + xy] : a[((size_t)i * K + k) * XY + xy];
          cf bv = conjB ? b[((size_t)j * K + k) * XY + xy] : b[((size_t)k * J + j) * XY + xy];
          if (conjA)
            acc = conj(av) * bv + acc;
          else if (conjB)
            acc = av * conj(bv) + acc;
          else
            acc = av * bv + acc;
        }
        acc.re *= invNorm;
        acc.im *= invNorm;
        c[((size_t)i * J + j) * XY + xy] = acc;
      }
    }
  }
}

// FFTIteratedConvolution<N> (FFTIteratedConvolution.cuh:624-755), the three
// kernels at :97-207 (pass 0), :254-363 (pass 1), :409-524 (pass 2).
// ins/outs are host arrays of numTiles descriptors whose data pointers are host
// pointers.  weight is [Cout][Cin][kH][kW] with the given strides.
// Returns 1 if the pass code matched (the reference's "true"), else 0.
int orc_iterated_conv(int N, const void* insV, const void* outsV, float* weight,
                      const int* wSize, const int* wStride, int pass, float scale,
                      int batchSize, int numTiles) {
  if (!(N == 8 || N == 16 || N == 32)) return 0;
  const TileDesc* ins = static_cast<const TileDesc*>(insV);
  const TileDesc* outs = static_cast<const TileDesc*>(outsV);
  TileDesc wt;
  wt.padL = 0;
  wt.padU = 0;
  wt.data = weight;
  for (int d = 0; d < 4; ++d) {
    wt.size[d] = wSize[d];
    wt.stride[d] = wStride[d];
  }
  const int H = N / 2;
  const int Cout = wSize[0], Cin = wSize[1];
  const float invNorm = 1.0f / (float)(N * N);

  auto packedProduct = [&](const cf* p, const cf* q, cf* acc, bool conjQ) {
    // rows 1..N/2-1: plain products; row 0 carries two real-row spectra
    // (FFTIteratedConvolution.cuh:161-186 and :318-343)
    for (int x = 0; x < N; ++x) {
      if (x > 0) {
        cf p0, pN2, q0, qN2;
        unpackRow0(p, N, x, &p0, &pN2);
        unpackRow0(q, N, x, &q0, &qN2);
        cf r0 = conjQ ? p0 * conj(q0) : p0 * q0;
        cf rN2 = conjQ ? pN2 * conj(qN2) : pN2 * qN2;
        acc[x] = acc[x] + (r0 + swp(conj(rN2)));
      } else {
        acc[0] = acc[0] + mk(p[0].re * q[0].re, p[0].im * q[0].im);
      }
    }
    for (int i = 1; i < H; ++i)
      for (int x = 0; x < N; ++x) {
        cf pv = p[i * N + x], qv = q[i * N + x];
        acc[i * N + x] = acc[i * N + x] + (conjQ ? pv * conj(qv) : pv * qv);
      }
  };

  if (pass == 0) {  // FFT_UpdateOutput
#pragma omp parallel for collapse(3) schedule(dynamic)
    for (int t = 0; t < numTiles; ++t)
      for (int n = 0; n < batchSize; ++n)
        for (int f = 0; f < Cout; ++f) {
          if (n >= ins[t].size[0]) continue;
          std::vector<cf> acc((size_t)H * N, mk(0.0f)), wei((size_t)H * N), inp((size_t)H * N);
          for (int c = 0; c < Cin; ++c) {
            loadPackedTile(wei.data(), N, wt, f, c);
            coreForward(wei.data(), N);
            loadPackedTile(inp.data(), N, ins[t], n, c);
            coreForward(inp.data(), N);
            packedProduct(inp.data(), wei.data(), acc.data(), true);
          }
          coreInverse(acc.data(), N, true);
          storePackedTile(acc.data(), N, outs[t], n, f, invNorm);
        }
    return 1;
  }
  if (pass == 1) {  // FFT_UpdateGradInput
#pragma omp parallel for collapse(3) schedule(dynamic)
    for (int t = 0; t < numTiles; ++t)
      for (int n = 0; n < batchSize; ++n)
        for (int c = 0; c < Cin; ++c) {
          if (n >= ins[t].size[0]) continue;
          std::vector<cf> acc((size_t)H * N, mk(0.0f)), wei((size_t)H * N), out((size_t)H * N);
          for (int f = 0; f < Cout; ++f) {
            loadPackedTile(wei.data(), N, wt, f, c);
            coreForward(wei.data(), N);
            loadPackedTile(out.data(), N, outs[t], n, f);
            coreForward(out.data(), N);
            packedProduct(out.data(), wei.data(), acc.data(), false);
          }
          coreInverse(acc.data(), N, true);
          storePackedTile(acc.data(), N, ins[t], n, c, invNorm);
        }
    return 1;
  }
  if (pass == 2) {  // FFT_AccGradParameters
    const float invNormScale = scale / (float)(N * N);
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (int f = 0; f < Cout; ++f)
      for (int c = 0; c < Cin; ++c) {
        std::vector<cf> acc((size_t)(H + 1) * N, mk(0.0f)), out((size_t)(H + 1) * N),
            inp((size_t)(H + 1) * N);
        for (int t = 0; t < numTiles; ++t) {
          const int Bt = ins[t].size[0];
          for (int n = 0; n < Bt; ++n) {
            loadPackedTile(out.data(), N, outs[t], n, f);
            coreForward(out.data(), N);
            loadPackedTile(inp.data(), N, ins[t], n, c);
            coreForward(inp.data(), N);
            // rows 0 and N/2 are unpacked before the product (:475-497)
            for (int x = 0; x < N; ++x) {
              cf i0, iN2, o0, oN2;
              unpackRow0(inp.data(), N, x, &i0, &iN2);
              unpackRow0(out.data(), N, x, &o0, &oN2);
              acc[x] = acc[x] + i0 * conj(o0);
              acc[(size_t)H * N + x] = acc[(size_t)H * N + x] + iN2 * conj(oN2);
            }
            for (int i = 1; i < H; ++i)
              for (int x = 0; x < N; ++x)
                acc[i * N + x] = acc[i * N + x] + inp[i * N + x] * conj(out[i * N + x]);
          }
        }
        coreInverse(acc.data(), N, false);
        storePackedTile(acc.data(), N, wt, f, c, invNormScale);
      }
    return 1;
  }
  return 0;
}

// --------------------------- double precision ------------------------------

// out[b][k] = sum_x real[b][x] e^{-2 pi i k x / N}, k = 0..N/2
void ref64_dft1d_r2c(const float* real, int B, int N, double* out) {
  const int nc = N / 2 + 1;
#pragma omp parallel for schedule(static)
  for (int b = 0; b < B; ++b)
    for (int k = 0; k < nc; ++k) {
      double re = 0, im = 0;
      for (int x = 0; x < N; ++x) {
        double ang = -2.0 * M_PI * (double)((k * x) % N) / N;
        re += real[(size_t)b * N + x] * std::cos(ang);
        im += real[(size_t)b * N + x] * std::sin(ang);
      }
      out[((size_t)b * nc + k) * 2] = re;
      out[((size_t)b * nc + k) * 2 + 1] = im;
    }
}

// real[b][x] = sum_k c[b][k] e^{+2 pi i k x / N} over the Hermitian extension
// (unnormalised: gain N)
void ref64_idft1d_c2r(const float* cplx, int B, int N, double* out) {
  const int nc = N / 2 + 1;
#pragma omp parallel for schedule(static)
  for (int b = 0; b < B; ++b)
    for (int x = 0; x < N; ++x) {
      double acc = 0;
      for (int k = 0; k < N; ++k) {
        int m = k < nc ? k : N - k;
        double cr = cplx[((size_t)b * nc + m) * 2];
        double ci = cplx[((size_t)b * nc + m) * 2 + 1] * (k < nc ? 1.0 : -1.0);
        double ang = 2.0 * M_PI * (double)((k * x) % N) / N;
        acc += cr * std::cos(ang) - ci * std::sin(ang);
      }
      out[(size_t)b * N + x] = acc;
    }
}

// F[ky][kx] = sum_{y,x} X[y][x] e^{-2 pi i (ky y + kx x)/N}, X = real placed at
// (padU, padL) of a zero N x N plane.
// layout 0: out[b][ky][kx], ky = 0..N/2   (the N <= 32 convention)
// layout 1: out[b][kx][ky], kx = 0..N/2   (the N >= 64 convention)
void ref64_dft2d_r2c(const float* real, int B, int h, int w, int N, int padL, int padU,
                     int layout, double* out) {
  const int nc = N / 2 + 1;
  std::vector<double> cs(N), sn(N);
  for (int i = 0; i < N; ++i) {
    cs[i] = std::cos(-2.0 * M_PI * i / N);
    sn[i] = std::sin(-2.0 * M_PI * i / N);
  }
#pragma omp parallel for schedule(static)
  for (int b = 0; b < B; ++b) {
    std::vector<double> X((size_t)N * N, 0.0);
    for (int y = 0; y < N; ++y)
      for (int x = 0; x < N; ++x)
        if (inBounds2(y, x, padU, padL, h, w))
          X[(size_t)y * N + x] = real[((size_t)b * h + (y - padU)) * w + x - padL];
    // rows first: G[y][kx]
    std::vector<double> Gr((size_t)N * N), Gi((size_t)N * N);
    for (int y = 0; y < N; ++y)
      for (int kx = 0; kx < N; ++kx) {
        double re = 0, im = 0;
        for (int x = 0; x < N; ++x) {
          int m = (kx * x) % N;
          re += X[(size_t)y * N + x] * cs[m];
          im += X[(size_t)y * N + x] * sn[m];
        }
        Gr[(size_t)y * N + kx] = re;
        Gi[(size_t)y * N + kx] = im;
      }
    for (int ky = 0; ky < N; ++ky)
      for (int kx = 0; kx < N; ++kx) {
        if (layout == 0 ? ky >= nc : kx >= nc) continue;
        double re = 0, im = 0;
        for (int y = 0; y < N; ++y) {
          int m = (ky * y) % N;
          double gr = Gr[(size_t)y * N + kx], gi = Gi[(size_t)y * N + kx];
          re += gr * cs[m] - gi * sn[m];
          im += gr * sn[m] + gi * cs[m];
        }
        size_t idx = layout == 0 ? ((size_t)b * nc + ky) * N + kx : ((size_t)b * nc + kx) * N + ky;
        out[idx * 2] = re;
        out[idx * 2 + 1] = im;
      }
  }
}

// Valid cross-correlation (no kernel flip):
// out[n][f][y][x] = sum_{c,u,v} in[n][c][y+u][x+v] * w[f][c][u][v]
void ref64_corr2d_valid(const float* in, const float* w, int Nb, int Cin, int H, int W,
                        int Cout, int kH, int kW, double* out) {
  const int oH = H - kH + 1, oW = W - kW + 1;
#pragma omp parallel for collapse(2) schedule(static)
  for (int n = 0; n < Nb; ++n)
    for (int f = 0; f < Cout; ++f)
      for (int y = 0; y < oH; ++y)
        for (int x = 0; x < oW; ++x) {
          double acc = 0;
          for (int c = 0; c < Cin; ++c)
            for (int u = 0; u < kH; ++u)
              for (int v = 0; v < kW; ++v)
                acc += (double)in[(((size_t)n * Cin + c) * H + y + u) * W + x + v] *
                       (double)w[(((size_t)f * Cin + c) * kH + u) * kW + v];
          out[(((size_t)n * Cout + f) * oH + y) * oW + x] = acc;
        }
}

// Same sum restricted to a list of output coordinates (n, f, y, x) so that very
// large configurations can be spot-checked.
void ref64_corr2d_valid_at(const float* in, const float* w, int Cin, int H, int W, int kH,
                           int kW, const int* coords, int ncoords, double* out) {
#pragma omp parallel for schedule(static)
  for (int i = 0; i < ncoords; ++i) {
    const int n = coords[4 * i], f = coords[4 * i + 1], y = coords[4 * i + 2], x = coords[4 * i + 3];
    double acc = 0;
    for (int c = 0; c < Cin; ++c)
      for (int u = 0; u < kH; ++u)
        for (int v = 0; v < kW; ++v)
          acc += (double)in[(((size_t)n * Cin + c) * H + y + u) * W + x + v] *
                 (double)w[(((size_t)f * Cin + c) * kH + u) * kW + v];
    out[i] = acc;
  }
}

// gradInput of the valid correlation: gin[n][c][y][x] = sum_{f,u,v} gout[n][f][y-u][x-v] w[f][c][u][v]
void ref64_corr2d_grad_input(const float* gout, const float* w, int Nb, int Cin, int H, int W,
                             int Cout, int kH, int kW, double* gin) {
  const int oH = H - kH + 1, oW = W - kW + 1;
#pragma omp parallel for collapse(2) schedule(static)
  for (int n = 0; n < Nb; ++n)
    for (int c = 0; c < Cin; ++c)
      for (int y = 0; y < H; ++y)
        for (int x = 0; x < W; ++x) {
          double acc = 0;
          for (int f = 0; f < Cout; ++f)
            for (int u = 0; u < kH; ++u)
              for (int v = 0; v < kW; ++v) {
                int oy = y - u, ox = x - v;
                if (oy < 0 || oy >= oH || ox < 0 || ox >= oW) continue;
                acc += (double)gout[(((size_t)n * Cout + f) * oH + oy) * oW + ox] *
                       (double)w[(((size_t)f * Cin + c) * kH + u) * kW + v];
              }
          gin[(((size_t)n * Cin + c) * H + y) * W + x] = acc;
        }
}

// gradWeight: gw[f][c][u][v] = sum_{n,y,x} in[n][c][y+u][x+v] gout[n][f][y][x]
void ref64_corr2d_grad_weight(const float* in, const float* gout, int Nb, int Cin, int H, int W,
                              int Cout, int kH, int kW, double* gw) {
  const int oH = H - kH + 1, oW = W - kW + 1;
#pragma omp parallel for collapse(2) schedule(static)
  for (int f = 0; f < Cout; ++f)
    for (int c = 0; c < Cin; ++c)
      for (int u = 0; u < kH; ++u)
        for (int v = 0; v < kW; ++v) {
          double acc = 0;
          for (int n = 0; n < Nb; ++n)
            for (int y = 0; y < oH; ++y)
              for (int x = 0; x < oW; ++x)
                acc += (double)in[(((size_t)n * Cin + c) * H + y + u) * W + x + v] *
                       (double)gout[(((size_t)n * Cout + f) * oH + y) * oW + x];
          gw[(((size_t)f * Cin + c) * kH + u) * kW + v] = acc;
        }
}

// The same two gradients restricted to lists of coordinates, so that layers too large for
// the full sums can be spot-checked: (n, c, y, x) of gradInput, (f, c, u, v) of gradWeight.
void ref64_corr2d_grad_input_at(const float* gout, const float* w, int Cin, int H, int W, int Cout,
                                int kH, int kW, const int* coords, int ncoords, double* out) {
  const int oH = H - kH + 1, oW = W - kW + 1;
#pragma omp parallel for schedule(static)
  for (int i = 0; i < ncoords; ++i) {
    const int n = coords[4 * i], c = coords[4 * i + 1], y = coords[4 * i + 2], x = coords[4 * i + 3];
    double acc = 0;
    for (int f = 0; f < Cout; ++f)
      for (int u = 0; u < kH; ++u) {
        const int oy = y - u;
        if (oy < 0 || oy >= oH) continue;
        for (int v = 0; v < kW; ++v) {
          const int ox = x - v;
          if (ox < 0 || ox >= oW) continue;
          acc += (double)gout[(((size_t)n * Cout + f) * oH + oy) * oW + ox] *
                 (double)w[(((size_t)f * Cin + c) * kH + u) * kW + v];
        }
      }
    out[i] = acc;
  }
}

void ref64_corr2d_grad_weight_at(const float* in, const float* gout, int Nb, int Cin, int H, int W,
                                 int Cout, int kH, int kW, const int* coords, int ncoords,
                                 double* out) {
  const int oH = H - kH + 1, oW = W - kW + 1;
#pragma omp parallel for schedule(dynamic)
  for (int i = 0; i < ncoords; ++i) {
    const int f = coords[4 * i], c = coords[4 * i + 1], u = coords[4 * i + 2], v = coords[4 * i + 3];
    double acc = 0;
    for (int n = 0; n < Nb; ++n)
      for (int y = 0; y < oH; ++y) {
        const float* ir = in + (((size_t)n * Cin + c) * H + y + u) * W + v;
        const float* gr = gout + (((size_t)n * Cout + f) * oH + y) * oW;
        for (int x = 0; x < oW; ++x) acc += (double)ir[x] * (double)gr[x];
      }
    out[i] = acc;
  }
}

// fp64 contraction with the transposeMM semantics (no invNorm on the
// accumulated-into value: pure sum, scaled)
void ref64_transpose_mm(const float* A, const float* B, double* C, int I, int J, int K, int XY,
                        int conjA, int conjB, double invNorm) {
#pragma omp parallel for collapse(2) schedule(static)
  for (int i = 0; i < I; ++i)
    for (int j = 0; j < J; ++j)
      for (int xy = 0; xy < XY; ++xy) {
        double re = 0, im = 0;
        for (int k = 0; k < K; ++k) {
          size_t ia = conjA ? ((size_t)k * I + i) * XY + xy : ((size_t)i * K + k) * XY + xy;
          size_t ib = conjB ? ((size_t)j * K + k) * XY + xy : ((size_t)k * J + j) * XY + xy;
          double ar = A[2 * ia], ai = A[2 * ia + 1] * (conjA ? -1.0 : 1.0);
          double br = B[2 * ib], bi = B[2 * ib + 1] * (conjB ? -1.0 : 1.0);
          re += ar * br - ai * bi;
          im += ar * bi + ai * br;
        }
        C[(((size_t)i * J + j) * XY + xy) * 2] = re * invNorm;
        C[(((size_t)i * J + j) * XY + xy) * 2 + 1] = im * invNorm;
      }
}

}  // extern "C"
