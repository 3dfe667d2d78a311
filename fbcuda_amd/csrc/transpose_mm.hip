// Per-frequency complex contraction on the fp32 matrix cores (replaces
// transposeMMTiledKernelUnrolled / ...Small / the generic fallback,
// MM-inl.cuh:34-506, and the dispatch at :515-814).
//
//   C[i][j][xy] = invNorm * ((accumulate ? C[i][j][xy] : 0) + sum_k opA[i][k][xy] * opB[k][j][xy])
//
// Operands keep the reference layout: complex, xy innermost and contiguous, so
// xy is the batch index of 'XY' independent small GEMMs and a coalesced global
// access is a run of consecutive bins of one (row, col) element.
//
// A workgroup (4 waves) owns a 32 x 32 tile of C for 16 consecutive bins (one
// 128-byte line per element).  Per 4-deep slice of k it stages opA and opB in
// LDS split into real and imaginary planes [bin][k][row], conjugation folded
// into the sign of the imaginary plane, while the next slice is already in
// flight in registers.  Wave w then runs bins 4w..4w+3 with
// v_mfma_f32_32x32x2_f32: four real products per complex product,
//   Cre += Ar*Br + (-Ai)*Bi,   Cim += Ar*Bi + Ai*Br,
// 128 accumulator registers per lane.  Only this contraction uses MFMA; it is
// the one dense product of the convolution path.
#include "common.h"

namespace fbfft_amd {
namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int TI = 32, TJ = 32, XB = 16, KC = 4, THREADS = 256;  // 4 waves
constexpr int XS = KC * 32 + 4;              // bin stride of an LDS plane (dwords), padded
constexpr int PLANE = XB * XS;               // one of Ar, Ai, Br, Bi
constexpr int CSTR = XB + 1;                 // padded bin stride of the C staging buffer (complex)
constexpr int LDS_FLOATS = (4 * PLANE > 8 * 32 * CSTR * 2) ? 4 * PLANE : 8 * 32 * CSTR * 2;

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

// 16 bins x 4 k x 32 rows of one operand: each lane fetches two float4 (bins
// 2p, 2p+1 of two (row, k) elements).  Lanes of a wave: p = lane % 8 walks the
// line, lane / 8 walks 8 consecutive rows.
struct Fetch {
  float4 v[2];
};

template <bool VEC4>
__device__ __forceinline__ Fetch fetchSlice(const float* base, long rowStride, long kStride,
                                            int rows, int row0, int K, int k0, int XY, int x0,
                                            int t) {
  Fetch f;
  const int p = t % 8;
  const int x = x0 + 2 * p;
  f.v[0] = float4{0.f, 0.f, 0.f, 0.f};
  f.v[1] = float4{0.f, 0.f, 0.f, 0.f};
  // element e = lane/8 + 32u -> row = e % 32, kk = e / 32: one call covers two
  // values of k; the caller issues a second call for k0 + 2
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int e = t / 8 + 32 * u;
    const int r = e % 32;
    const int kk = e / 32;  // 0 or 1 (+2 by the caller through k0)
    const int row = row0 + r, k = k0 + kk;
    if (row < rows && k < K && x < XY) {
      const float* src = base + (long)row * rowStride + (long)k * kStride + 2L * x;
      if (VEC4 && x + 1 < XY) {
        f.v[u] = *reinterpret_cast<const float4*>(src);
      } else {
        float2 a = *reinterpret_cast<const float2*>(src);
        f.v[u].x = a.x;
        f.v[u].y = a.y;
        if (x + 1 < XY) {
          float2 b = *reinterpret_cast<const float2*>(src + 2);
          f.v[u].z = b.x;
          f.v[u].w = b.y;
        }
      }
    }
  }
  return f;
}

__device__ __forceinline__ void stashSlice(float* re, float* im, const Fetch& f, float sign, int kBase,
                                           int t) {
  const int p = t % 8;
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int e = t / 8 + 32 * u;
    const int r = e % 32, kk = kBase + e / 32;
    const int o = kk * 32 + r;
    re[(2 * p) * XS + o] = f.v[u].x;
    im[(2 * p) * XS + o] = sign * f.v[u].y;
    re[(2 * p + 1) * XS + o] = f.v[u].z;
    im[(2 * p + 1) * XS + o] = sign * f.v[u].w;
  }
}

template <bool VEC4>
__global__ __launch_bounds__(THREADS, 2) void transposeMMKernel(MMArgs a) {
  __shared__ __align__(8) float lds[LDS_FLOATS];
  float* Ar = lds;
  float* Ai = lds + PLANE;
  float* Br = lds + 2 * PLANE;
  float* Bi = lds + 3 * PLANE;

  const int t = threadIdx.x;
  const int lane = t % 64, w = t / 64;
  // Workgroups are dealt round-robin to the 8 XCDs, each with its own L2.  Give
  // every XCD a contiguous range of logical ids, ordered bin-chunk first, so that
  // all (i, j) tiles that re-read the same lines of A and B share one L2.
  const int tilesJ = (a.J + TJ - 1) / TJ, tilesI = (a.I + TI - 1) / TI;
  const int total = a.chunks * tilesI * tilesJ;
  const int per = (total + 7) / 8;
  const int logical = (blockIdx.x % 8) * per + blockIdx.x / 8;
  if (logical >= total) return;
  const int x0 = (logical / (tilesI * tilesJ)) * XB;
  const int rem = logical % (tilesI * tilesJ);
  const int j0 = (rem % tilesJ) * TJ;
  const int i0 = (rem / tilesJ) * TI;

  floatx16 cre[4], cim[4];
#pragma unroll
  for (int b = 0; b < 4; ++b)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      cre[b][r] = 0.f;
      cim[b][r] = 0.f;
    }

  // slice = KC = 4 values of k: two fetches (k0, k0+1) and (k0+2, k0+3) per operand
  Fetch fa0, fa1, fb0, fb1;
  auto fetchAll = [&](int k0) {
    fa0 = fetchSlice<VEC4>(a.A, a.aRow, a.aK, a.I, i0, a.K, k0, a.XY, x0, t);
    fa1 = fetchSlice<VEC4>(a.A, a.aRow, a.aK, a.I, i0, a.K, k0 + 2, a.XY, x0, t);
    fb0 = fetchSlice<VEC4>(a.B, a.bCol, a.bK, a.J, j0, a.K, k0, a.XY, x0, t);
    fb1 = fetchSlice<VEC4>(a.B, a.bCol, a.bK, a.J, j0, a.K, k0 + 2, a.XY, x0, t);
  };
  fetchAll(0);
  for (int k0 = 0; k0 < a.K; k0 += KC) {
    __syncthreads();  // previous slice fully consumed
    stashSlice(Ar, Ai, fa0, a.aSign, 0, t);
    stashSlice(Ar, Ai, fa1, a.aSign, 2, t);
    stashSlice(Br, Bi, fb0, a.bSign, 0, t);
    stashSlice(Br, Bi, fb1, a.bSign, 2, t);
    __syncthreads();
    if (k0 + KC < a.K) fetchAll(k0 + KC);
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const int xo = (4 * w + b) * XS;
#pragma unroll
      for (int s = 0; s < KC / 2; ++s) {
        // lane supplies row/col lane%32 at k = 2s + lane/32: 64 consecutive dwords
        const int o = xo + s * 64 + lane;
        const float ar = Ar[o], ai = Ai[o], br = Br[o], bi = Bi[o];
        cre[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(ar, br, cre[b], 0, 0, 0);
        cre[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(-ai, bi, cre[b], 0, 0, 0);
        cim[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(ar, bi, cim[b], 0, 0, 0);
        cim[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(ai, br, cim[b], 0, 0, 0);
      }
    }
  }

  // ---- epilogue: C leaves through LDS so that every store covers whole 128-byte
  // runs (the 16 bins of one (i, j) element); written straight from the
  // accumulators each lane would scatter 8-byte pieces 4 KB apart.
  // Register r of lane l holds row 8*(r/4) + 4*(l/32) + r%4, column l%32, so the
  // four registers 4c..4c+3 of all lanes form rows 8c..8c+7: one chunk.
  float2* stage = reinterpret_cast<float2*>(lds);  // [8 rows][32 cols][CSTR] complex
  const int col = lane % 32, hh = lane / 32;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    __syncthreads();  // operand slices / previous chunk fully consumed
#pragma unroll
    for (int rr = 0; rr < 4; ++rr) {
      const int row = 4 * hh + rr;
#pragma unroll
      for (int b = 0; b < 4; ++b)
        stage[(row * 32 + col) * CSTR + 4 * w + b] = float2{cre[b][4 * c + rr], cim[b][4 * c + rr]};
    }
    __syncthreads();
    // 256 (row, col) elements x 16 bins: 16 lanes per element, 16 elements per pass
    const int xl = t % 16;
#pragma unroll
    for (int pass = 0; pass < 16; ++pass) {
      const int e = t / 16 + 16 * pass;  // 0..255
      const int row = e / 32, cc = e % 32;
      const int i = i0 + 8 * c + row, j = j0 + cc, x = x0 + xl;
      if (i < a.I && j < a.J && x < a.XY) {
        float2 acc = stage[(row * 32 + cc) * CSTR + xl];
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

}  // namespace

// A, B, C: complex-as-float views collapsed to [d0][d1][xy][2] with unit xy
// stride; s0/s1 are the float strides of the first two dimensions.
int launchTransposeMM(const float* A, long a0, long a1, const float* B, long b0, long b1, float* C,
                      long c0, long c1, int I, int J, int K, int XY, bool conjA, bool conjB,
                      bool accumulate, float invNorm, hipStream_t s) {
  if (I <= 0 || J <= 0 || XY <= 0) return FBFFT_SUCCESS;
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
  m.chunks = ceilDiv(XY, XB);
  const int total = m.chunks * ceilDiv(J, TJ) * ceilDiv(I, TI);
  dim3 grid((total + 7) / 8 * 8), block(THREADS);
  const bool vec4 = aligned(A, 16) && aligned(B, 16) && a0 % 4 == 0 && a1 % 4 == 0 &&
                    b0 % 4 == 0 && b1 % 4 == 0;
  if (vec4)
    transposeMMKernel<true><<<grid, block, 0, s>>>(m);
  else
    transposeMMKernel<false><<<grid, block, 0, s>>>(m);
  return launchStatus();
}

}  // namespace fbfft_amd
