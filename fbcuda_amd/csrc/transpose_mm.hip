// Per-frequency complex contraction on the fp32 matrix cores (replaces
// transposeMMTiledKernelUnrolled / ...Small / the generic fallback,
// MM-inl.cuh:34-506, and the dispatch at :515-814).
//
//   C[i][j][xy] = invNorm * ((accumulate ? C[i][j][xy] : 0) + sum_k opA[i][k][xy] * opB[k][j][xy])
//
// Operands keep the reference layout: complex, xy innermost and contiguous, so
// xy is the batch index of 'XY' independent small GEMMs and a coalesced global
// access is a run of consecutive bins of one (row, col) element.  Accumulators
// are needed for every bin of a run at once, which bounds the tile: a workgroup
// of 8 waves owns a 64 x 64 tile of C for 8 consecutive bins (64-byte runs; the
// other half of each line goes to the neighbouring workgroup on the same XCD),
// wave w owning bin w: 4 MFMA 32x32 sub-tiles x 3 partial products = 192
// accumulator registers per lane.
//
// Per 4-deep slice of k the workgroup stages opA and opB in LDS split into real
// and imaginary planes [bin][k][row] (conjugation folded into the sign of the
// imaginary plane), two buffers deep, while the slice after next is in flight in
// registers; each
// wave then issues v_mfma_f32_32x32x2_f32, three real products per complex
// product (k1 = (Ar+Ai) Br, k2 = Ar (Bi-Br), k3 = Ai (Br+Bi); Cre = k1 - k3,
// Cim = k1 + k2).  C leaves through LDS
// so that stores cover whole runs.  Only this contraction uses MFMA; it is the
// one dense product of the convolution path.
//
// Packed spectra (fbfft_transpose_mm_packed): operands [..][..][N/2][N] whose row 0
// holds P[x] = F0[x] + i FH[x], the spectra of the two real rows 0 and N/2 of an
// N x N transform (the Unpack = false format of fbfft/FFT2D32.cuh:421-427).  Rows
// 1 .. N/2-1 are plain bins and go through the kernel above.  Row 0 follows the
// product rule of fbfft/FFTIteratedConvolution.cuh:161-186: unpack both operands,
// multiply F0 with F0 and FH with FH, re-pack.  The PACKED0 variant of the kernel
// does that on the way into and out of LDS: a workgroup takes four x (0 < x < N/2)
// and its eight waves own the "virtual bins" F0[x] and FH[x], computed from P[x] and
// P[N-x] when a slice is parked; the epilogue combines C0[x] and CH[x] into P[x] and
// P[N-x].  x = 0 pairs with x = N/2: both hold two real values, which multiply
// component by component (no cross terms).
#include "common.h"

namespace fbfft_amd {
namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int TI = 64, TJ = 64, XB = 8, KC = 4, THREADS = 512;  // 8 waves, one bin each
constexpr int XS = KC * 64 + 4;   // bin stride of an LDS plane (dwords): the 4 bin pairs a
                                  // half-wave writes land 8 banks apart
constexpr int PLANE = XB * XS;    // one of Ar, Ai, Br, Bi
constexpr int CSTR = XB + 1;      // padded bin stride of the C staging buffer (complex)
constexpr int STAGE_FLOATS = 8 * TJ * CSTR * 2;
constexpr int BUF = 4 * PLANE;    // Ar, Ai, Br, Bi of one slice
constexpr int LDS_FLOATS = (2 * BUF > STAGE_FLOATS) ? 2 * BUF : STAGE_FLOATS;

struct MMArgs {
  const float* A;
  const float* B;
  float* C;
  int I, J, K, XY;
  // strides in floats of the row / col / k dimension as seen through op()
  long aRow, aK;   // opA[i][k] = A[i*aRow + k*aK]
  long bK, bCol;   // opB[k][j] = B[k*bK + j*bCol]
  long cRow, cCol;
  float aSign, bSign;  // -1 when the operand is conjugated
  float invNorm;
  int accumulate;
  int chunks;  // ceil(XY / XB)
};

// One slice of one operand: 64 rows x KC k x 8 bins.  Lane t fetches bins 2p, 2p+1
// (p = t % 4) of row (t/4) % 64 at k = (t/4)/64 + 2u: within a wave
// 16 consecutive rows, 64 bytes each.
struct Fetch {
  float4 v[KC / 2];
};

// Every load is issued unconditionally at an address clamped into the operand; the
// values outside it are zeroed only when the slice is parked in LDS one iteration
// later, so nothing waits for a load between its issue and the products of the
// current slice.  VEC4 additionally needs XY even (a bin pair never straddles the end).
// bin that shares its two spectra with bin x of a packed row 0
__device__ __forceinline__ int packedPartner(int x, int N) { return x == 0 ? N / 2 : N - x; }

// PACKED0: XY is the length N of packed row 0, x0 a multiple of 4 below N/2; lane
// t fetches P[x] and P[partner(x)] for x = x0 + t % 4.
template <bool VEC4, bool PACKED0>
__device__ __forceinline__ Fetch fetchSlice(const float* base, long rowStride, long kStride,
                                            int rows, int row0, int K, int k0, int XY, int x0,
                                            int t) {
  Fetch f;
  const int p = t % 4;
  if constexpr (PACKED0) {
    const int e = t / 4;
    const int row = row0 + e % 64;
    const int x = x0 + p;
    const float* src0 = base + (long)min(row, rows - 1) * rowStride;
    const long o1 = 2L * x, o2 = 2L * packedPartner(x, XY);
#pragma unroll
    for (int u = 0; u < KC / 2; ++u) {
      const int k = k0 + e / 64 + 2 * u;
      const float* src = src0 + (long)min(k, K - 1) * kStride;
      const float2 a = *reinterpret_cast<const float2*>(src + o1);
      const float2 b = *reinterpret_cast<const float2*>(src + o2);
      f.v[u] = float4{a.x, a.y, b.x, b.y};
    }
    return f;
  }
  const int x = x0 + 2 * p;
  const int e = t / 4;
  const int row = row0 + e % 64;
  const float* src0 = base + (long)min(row, rows - 1) * rowStride + 2L * min(x, XY - (VEC4 ? 2 : 1));
  const long x1off = x + 1 < XY ? 2 : 0;
#pragma unroll
  for (int u = 0; u < KC / 2; ++u) {
    const int k = k0 + e / 64 + 2 * u;
    const float* src = src0 + (long)min(k, K - 1) * kStride;
    if constexpr (VEC4) {
      f.v[u] = *reinterpret_cast<const float4*>(src);
    } else {
      const float2 a = *reinterpret_cast<const float2*>(src);
      const float2 b = *reinterpret_cast<const float2*>(src + x1off);
      f.v[u] = float4{a.x, a.y, b.x, b.y};
    }
  }
  return f;
}

// Parks a fetched slice (k0 .. k0 + KC) in its LDS planes, zeroing what lies outside
// the operand.
template <bool PACKED0>
__device__ __forceinline__ void stashSlice(float* re, float* im, const Fetch& f, float sign,
                                           int rows, int row0, int K, int k0, int XY, int x0,
                                           int t) {
  const int p = t % 4;
  const int e = t / 4;
  if constexpr (PACKED0) {
    // virtual bin p: F0[x], virtual bin 4 + p: FH[x]; for x = 0 the two bins hold the
    // real pairs (F0[0], F0[N/2]) and (FH[0], FH[N/2]), which conjugation leaves alone
    const bool ok0 = row0 + e % 64 < rows;
    const bool ends = x0 + p == 0;
#pragma unroll
    for (int u = 0; u < KC / 2; ++u) {
      const int o = (e / 64 + 2 * u) * 64 + e % 64;
      const bool ok = ok0 && k0 + e / 64 + 2 * u < K;
      const float4 v = f.v[u];  // P[x] = (v.x, v.y), P[partner] = (v.z, v.w)
      const float r0 = ends ? v.x : 0.5f * (v.x + v.z);
      const float i0 = ends ? v.z : sign * 0.5f * (v.y - v.w);
      const float rH = ends ? v.y : 0.5f * (v.y + v.w);
      const float iH = ends ? v.w : sign * 0.5f * (v.z - v.x);
      re[p * XS + o] = ok ? r0 : 0.f;
      im[p * XS + o] = ok ? i0 : 0.f;
      re[(4 + p) * XS + o] = ok ? rH : 0.f;
      im[(4 + p) * XS + o] = ok ? iH : 0.f;
    }
    return;
  }
  const int x = x0 + 2 * p;
  const bool ok0 = row0 + e % 64 < rows && x < XY;
  const bool okX1 = x + 1 < XY;
#pragma unroll
  for (int u = 0; u < KC / 2; ++u) {
    const int o = (e / 64 + 2 * u) * 64 + e % 64;
    const bool ok = ok0 && k0 + e / 64 + 2 * u < K;
    re[(2 * p) * XS + o] = ok ? f.v[u].x : 0.f;
    im[(2 * p) * XS + o] = ok ? sign * f.v[u].y : 0.f;
    re[(2 * p + 1) * XS + o] = ok && okX1 ? f.v[u].z : 0.f;
    im[(2 * p + 1) * XS + o] = ok && okX1 ? sign * f.v[u].w : 0.f;
  }
}

// one workgroup's share: work item `logical` of a (PACKED0: of the packed row 0 of a)
template <bool VEC4, bool PACKED0>
__device__ __forceinline__ void transposeMMBody(const MMArgs& a, int logical, float* lds) {
  const int t = threadIdx.x;
  const int lane = t % 64, w = t / 64;
  const int tilesJ = (a.J + TJ - 1) / TJ, tilesI = (a.I + TI - 1) / TI;
  const int x0 = (logical / (tilesI * tilesJ)) * (PACKED0 ? XB / 2 : XB);
  const int rem = logical % (tilesI * tilesJ);
  // PACKED0: the waves holding the real pairs of x = 0 multiply component by component
  const bool ends = PACKED0 && x0 == 0 && w % 4 == 0;
  const float cross = ends ? 0.f : 1.f;
  const int j0 = (rem % tilesJ) * TJ;
  const int i0 = (rem / tilesJ) * TI;

  // sub-tile (si, sj): rows 32*si.., columns 32*sj...  Three real products per complex
  // product: with a = ar + i ai, b = br + i bi (conjugation already in the sign of
  // the imaginary planes), a b = (k1 - k3) + i (k1 + k2) for
  //   k1 = (ar + ai) br,  k2 = ar (bi - br),  k3 = ai (br + bi).
  floatx16 k1[2][2], k2[2][2], k3[2][2];
#pragma unroll
  for (int si = 0; si < 2; ++si)
#pragma unroll
    for (int sj = 0; sj < 2; ++sj)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        k1[si][sj][r] = 0.f;
        k2[si][sj][r] = 0.f;
        k3[si][sj][r] = 0.f;
      }

  Fetch fa, fb;
  auto fetchAll = [&](int k0) __attribute__((always_inline)) {
    fa = fetchSlice<VEC4, PACKED0>(a.A, a.aRow, a.aK, a.I, i0, a.K, k0, a.XY, x0, t);
    fb = fetchSlice<VEC4, PACKED0>(a.B, a.bCol, a.bK, a.J, j0, a.K, k0, a.XY, x0, t);
  };
  auto stashAll = [&](int buf, int k0) __attribute__((always_inline)) {
    float* base = lds + buf * BUF;
    stashSlice<PACKED0>(base, base + PLANE, fa, a.aSign, a.I, i0, a.K, k0, a.XY, x0, t);
    stashSlice<PACKED0>(base + 2 * PLANE, base + 3 * PLANE, fb, a.bSign, a.J, j0, a.K, k0, a.XY,
                        x0, t);
  };
  // Two slice buffers, one barrier per slice: while the waves multiply slice n out
  // of one buffer, each of them first parks slice n+1 (already in its registers) in
  // the other and requests slice n+2.
  if (a.K > 0) {  // with K = 0 the operands may have no memory behind them
    fetchAll(0);
    stashAll(0, 0);
    if (KC < a.K) fetchAll(KC);
  }
  __syncthreads();
  const int xo = w * XS + lane % 32 + 64 * (lane / 32);  // bin w, row/col lane%32, k parity lane/32
  int cur = 0;
  for (int k0 = 0; k0 < a.K; k0 += KC, cur ^= 1) {
    if (k0 + KC < a.K) {
      stashAll(cur ^ 1, k0 + KC);
      if (k0 + 2 * KC < a.K) fetchAll(k0 + 2 * KC);
    }
    const float* Ar = lds + cur * BUF;
    const float* Ai = Ar + PLANE;
    const float* Br = Ar + 2 * PLANE;
    const float* Bi = Ar + 3 * PLANE;
#pragma unroll
    for (int s = 0; s < KC / 2; ++s) {
      // the lane supplies row/col lane%32 (+32 for the second sub-tile) at k = 2s + lane/32
      const int o = xo + s * 128;
      float ar[2], ai[2], br[2], bi[2];
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        ar[q] = Ar[o + 32 * q];
        ai[q] = Ai[o + 32 * q];
        br[q] = Br[o + 32 * q];
        bi[q] = Bi[o + 32 * q];
      }
      float as[2], bd[2], bs[2];
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        if constexpr (PACKED0) {
          // real pairs: k1 = sum ar br and k3 = sum ai bi are the two results
          as[q] = __builtin_fmaf(cross, ai[q], ar[q]);
          bs[q] = __builtin_fmaf(cross, br[q], bi[q]);
        } else {
          as[q] = ar[q] + ai[q];
          bs[q] = br[q] + bi[q];
        }
        bd[q] = bi[q] - br[q];
      }
#pragma unroll
      for (int si = 0; si < 2; ++si)
#pragma unroll
        for (int sj = 0; sj < 2; ++sj) {
          k1[si][sj] = __builtin_amdgcn_mfma_f32_32x32x2f32(as[si], br[sj], k1[si][sj], 0, 0, 0);
          k2[si][sj] = __builtin_amdgcn_mfma_f32_32x32x2f32(ar[si], bd[sj], k2[si][sj], 0, 0, 0);
          k3[si][sj] = __builtin_amdgcn_mfma_f32_32x32x2f32(ai[si], bs[sj], k3[si][sj], 0, 0, 0);
        }
    }
    __syncthreads();  // slice k0 consumed by everybody, slice k0 + KC parked by everybody
  }

  // ---- epilogue: C leaves through LDS so that every store covers whole runs (the
  // 8 bins of one (i, j) element).  Register r of lane l holds row
  // 8*(r/4) + 4*(l/32) + r%4 and column l%32 of a sub-tile, so registers 4c..4c+3 of
  // all lanes form rows 8c..8c+7 of a sub-tile row: one chunk of 8 rows x 64 columns.
  float2* stage = reinterpret_cast<float2*>(lds);  // [8 rows][64 cols][CSTR] complex
  const int col = lane % 32, hh = lane / 32;
#pragma unroll
  for (int si = 0; si < 2; ++si)
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      __syncthreads();  // operand slices / previous chunk fully consumed
#pragma unroll
      for (int sj = 0; sj < 2; ++sj)
#pragma unroll
        for (int rr = 0; rr < 4; ++rr)
        {
          const float v1 = k1[si][sj][4 * c + rr], v2 = k2[si][sj][4 * c + rr],
                      v3 = k3[si][sj][4 * c + rr];
          stage[((4 * hh + rr) * TJ + 32 * sj + col) * CSTR + w] =
              ends ? float2{v1, v3} : float2{v1 - v3, v1 + v2};
        }
      __syncthreads();
      // 512 (row, col) elements x 8 bins: 8 lanes per element, 64 elements per pass
      const int xl = t % 8;
#pragma unroll
      for (int pass = 0; pass < 8; ++pass) {
        const int e = t / 8 + 64 * pass;  // 0..511
        const int row = e / TJ, cc = e % TJ;
        const int i = i0 + 32 * si + 8 * c + row, j = j0 + cc;
        int x = x0 + xl;
        float2 acc;
        if constexpr (PACKED0) {
          // lanes 0..3: P[x], lanes 4..7: P[partner(x)], from C0[x] and CH[x]
          const int q = xl % 4;
          const bool second = xl >= 4;
          const float2 c0 = stage[(row * TJ + cc) * CSTR + q];
          const float2 cH = stage[(row * TJ + cc) * CSTR + 4 + q];
          x = x0 + q;
          if (x == 0)
            acc = second ? float2{c0.y, cH.y} : float2{c0.x, cH.x};
          else
            acc = second ? float2{c0.x + cH.y, cH.x - c0.y} : float2{c0.x - cH.y, c0.y + cH.x};
          if (second) x = packedPartner(x, a.XY);
        } else {
          acc = stage[(row * TJ + cc) * CSTR + xl];
        }
        if (i < a.I && j < a.J && x < a.XY) {
          float* dst = a.C + (long)i * a.cRow + (long)j * a.cCol + 2L * x;
          if (a.accumulate) {
            float2 old = *reinterpret_cast<const float2*>(dst);
            acc.x += old.x;
            acc.y += old.y;
          }
          *reinterpret_cast<float2*>(dst) = float2{acc.x * a.invNorm, acc.y * a.invNorm};
        }
      }
    }
}

inline int workItems(const MMArgs& a) {
  return a.chunks * ((a.J + TJ - 1) / TJ) * ((a.I + TI - 1) / TI);
}

// Workgroups are dealt round-robin to the 8 XCDs, each with its own L2.  Every XCD
// gets a contiguous range of logical ids, ordered bin-chunk first, so that the tiles
// that re-read the same lines of A and B (and the two chunks that share a 128-byte
// line) meet in one L2.
__device__ __forceinline__ int logicalWorkItem(int total) {
  const int per = (total + 7) / 8;
  return (blockIdx.x % 8) * per + blockIdx.x / 8;
}

template <bool VEC4>
__global__ __launch_bounds__(THREADS) void transposeMMKernel(MMArgs a, int total) {
  __shared__ __align__(8) float lds[LDS_FLOATS];  // two slice buffers; later the C staging area
  const int logical = logicalWorkItem(total);
  if (logical < total) transposeMMBody<VEC4, false>(a, logical, lds);
}

// Packed spectra in one launch: work items [0, totalMain) are the plain bins of rows
// 1 .. N/2-1, the rest the chunks of packed row 0 - a handful of workgroups that would
// leave most of the chip idle in a launch of their own.
template <bool VEC4>
__global__ __launch_bounds__(THREADS) void transposeMMPackedKernel(MMArgs mainRows, int totalMain,
                                                                   MMArgs row0, int totalRow0) {
  __shared__ __align__(8) float lds[LDS_FLOATS];
  // every XCD takes its share of the (slower) row-0 items first, then its range of
  // plain items
  const int perRow0 = (totalRow0 + 7) / 8, perMain = (totalMain + 7) / 8;
  const int xcd = blockIdx.x % 8, slot = blockIdx.x / 8;
  if (slot < perRow0) {
    const int item = xcd * perRow0 + slot;
    if (item < totalRow0) transposeMMBody<false, true>(row0, item, lds);
  } else {
    const int item = xcd * perMain + slot - perRow0;
    if (slot - perRow0 < perMain && item < totalMain) transposeMMBody<VEC4, false>(mainRows, item, lds);
  }
}

MMArgs makeArgs(const float* A, long a0, long a1, const float* B, long b0, long b1, float* C,
                long c0, long c1, int I, int J, int K, int XY, bool conjA, bool conjB,
                bool accumulate, float invNorm, int chunks) {
  MMArgs m;
  m.A = A;
  m.B = B;
  m.C = C;
  m.I = I;
  m.J = J;
  m.K = K;
  m.XY = XY;
  // opA[i][k]: !conjA: A[i][k], conjA: conj(A[k][i]);  opB[k][j]: !conjB: B[k][j], conjB: conj(B[j][k])
  m.aRow = conjA ? a1 : a0;
  m.aK = conjA ? a0 : a1;
  m.bK = conjB ? b1 : b0;
  m.bCol = conjB ? b0 : b1;
  m.cRow = c0;
  m.cCol = c1;
  m.aSign = conjA ? -1.f : 1.f;
  m.bSign = conjB ? -1.f : 1.f;
  m.invNorm = invNorm;
  m.accumulate = accumulate ? 1 : 0;
  m.chunks = chunks;
  return m;
}

bool movesAsFloat4(const float* A, long a0, long a1, const float* B, long b0, long b1, int XY) {
  return aligned(A, 16) && aligned(B, 16) && a0 % 4 == 0 && a1 % 4 == 0 && b0 % 4 == 0 &&
         b1 % 4 == 0 && XY % 2 == 0;
}

}  // namespace

// A, B, C: complex-as-float views collapsed to [d0][d1][xy][2] with unit xy
// stride; s0/s1 are the float strides of the first two dimensions.
int launchTransposeMM(const float* A, long a0, long a1, const float* B, long b0, long b1, float* C,
                      long c0, long c1, int I, int J, int K, int XY, bool conjA, bool conjB,
                      bool accumulate, float invNorm, hipStream_t s) {
  if (I <= 0 || J <= 0 || XY <= 0) return FBFFT_SUCCESS;
  const MMArgs m = makeArgs(A, a0, a1, B, b0, b1, C, c0, c1, I, J, K, XY, conjA, conjB, accumulate,
                            invNorm, ceilDiv(XY, XB));
  const int total = workItems(m);
  dim3 grid((total + 7) / 8 * 8), block(THREADS);
  if (movesAsFloat4(A, a0, a1, B, b0, b1, XY))
    transposeMMKernel<true><<<grid, block, 0, s>>>(m, total);
  else
    transposeMMKernel<false><<<grid, block, 0, s>>>(m, total);
  return launchStatus();
}

// The same contraction on packed spectra [d0][d1][N/2][N][2]: rows 1 .. N/2-1 as
// plain bins, row 0 by the unpack / multiply / re-pack rule, all in one launch.
int launchTransposeMMPacked(const float* A, long a0, long a1, const float* B, long b0, long b1,
                            float* C, long c0, long c1, int I, int J, int K, int N, bool conjA,
                            bool conjB, bool accumulate, float invNorm, hipStream_t s) {
  if (I <= 0 || J <= 0) return FBFFT_SUCCESS;
  const int XY = (N / 2 - 1) * N;
  const MMArgs mainRows = makeArgs(A + 2 * N, a0, a1, B + 2 * N, b0, b1, C + 2 * N, c0, c1, I, J, K,
                                   XY, conjA, conjB, accumulate, invNorm, ceilDiv(XY, XB));
  // four x per workgroup, x < N/2
  const MMArgs row0 = makeArgs(A, a0, a1, B, b0, b1, C, c0, c1, I, J, K, N, conjA, conjB,
                               accumulate, invNorm, N / XB);
  const int totalMain = workItems(mainRows), totalRow0 = workItems(row0);
  dim3 grid(((totalMain + 7) / 8 + (totalRow0 + 7) / 8) * 8), block(THREADS);
  if (movesAsFloat4(A + 2 * N, a0, a1, B + 2 * N, b0, b1, XY))
    transposeMMPackedKernel<true><<<grid, block, 0, s>>>(mainRows, totalMain, row0, totalRow0);
  else
    transposeMMPackedKernel<false><<<grid, block, 0, s>>>(mainRows, totalMain, row0, totalRow0);
  return launchStatus();
}

}  // namespace fbfft_amd
