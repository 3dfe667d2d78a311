// FFT convolution forward pass (valid cross-correlation) as three kernels that
// hand spectra to each other in a layout chosen for the matrix cores.
//
// The reference's external callers run fbfft2D -> transposeMM -> fbifft2D on
// plane-major spectra [plane][bin] (MM-inl.cuh:188-196), which makes the
// frequency bin - the batch index of the contraction - the innermost dimension
// and caps the contraction's tile size (accumulators are needed for every bin of
// a cache line at once).  Here the spectra never take that shape:
//
//   1. forwardBinMajor:  planes -> S[bin][k][row]   (row = image / output plane)
//      a 256-lane workgroup transforms SLOTS = 512/N planes with consecutive
//      `row` and the same k and writes each bin as one contiguous run.
//   2. binGemm:          C[bin][i][j] = invNorm * sum_k A[bin][k][i] * conj(B[bin][k][j])
//      one workgroup = one bin x (128 x 64) tile; k-slices of A and B are
//      contiguous in HBM and are copied verbatim into LDS; 4 waves x 2 MFMA
//      32x32x2 sub-tiles x (re, im); every spectrum element is fetched from HBM
//      once per j-tile and C is written once with coalesced stores.  Workgroup
//      ids are remapped so that the j-tiles of a bin run on the same XCD (shared L2).
//   3. inverseBinMajor:  C[bin][i][j] -> planes, gathering runs of SLOTS
//      consecutive j per bin, inverse transform, crop on store.
//
// Spectra are unpacked (N/2+1 rows) so the contraction is a plain complex GEMM.
#include <stdlib.h>

#include "common.h"
#include "fft2d_core.h"
#include "fft_regs.h"

namespace fbfft_amd {
namespace {

constexpr int kT = 256;
typedef float floatx16 __attribute__((ext_vector_type(16)));

template <int N>
struct BMCfg {
  static constexpr int H = N / 2;
  static constexpr int T = N / 2;
  static constexpr int SLOTS = kT / T;                 // planes per workgroup
  static constexpr int RS = PlaneCfg<N>::RS;
  static constexpr int PSZ = (H + 1) * RS + 2;         // plane stride in LDS (complex), 16-byte aligned
  static constexpr int BINS = (H + 1) * N;
};

struct PlaneSet {
  float* base;      // plane (row, k) starts at base + row*sRow + k*sK
  long sRow, sK;
  int sy, sx, h, w;
  int R, K;         // valid rows / k
};

// ---- 1. planes -> S[bin][k][row] ----
template <int N>
__global__ __launch_bounds__(kT) void forwardBinMajor(PlaneSet ps, float2* S, int Rp, int Kp) {
  using C = BMCfg<N>;
  constexpr int H = C::H, T = C::T, SLOTS = C::SLOTS, RS = C::RS, PSZ = C::PSZ;
  __shared__ __align__(16) c32 lds[SLOTS * PSZ];
  const int t = threadIdx.x;
  const int s = t / T, l = t % T;
  const int r0 = blockIdx.x * SLOTS;
  const int k = blockIdx.y;
  const int row = r0 + s;

  c32 z0[H], z1[H];
  if (row < ps.R && k < ps.K) {
    loadColumnsWindow<N>(ps.base + (long)row * ps.sRow + (long)k * ps.sK, ps.sy, ps.sx, ps.h, ps.w,
                         0, 0, l, z0, z1);
  } else {
#pragma unroll
    for (int j = 0; j < H; ++j) z0[j] = z1[j] = c32{0.f, 0.f};
  }
  c32* plane = lds + s * PSZ;
  columnPassForward<N>(z0, z1, plane, l);
  __syncthreads();
  rowPassInPlace<N, true>(plane, l);
  __syncthreads();

  // lanes: sp = t % SLOTS walks the run (consecutive rows), bq = t / SLOTS walks bins
  const int sp = t % SLOTS, bq = t / SLOTS;
  const c32* src = lds + sp * PSZ;
  float2* dst = S + (long)k * Rp + r0 + sp;
  const long binStride = (long)Kp * Rp;
#pragma unroll 2
  for (int bin = bq; bin < C::BINS; bin += T) {
    const int r = bin / N, x = bin % N;
    c32 v;
    if (r == 0 || r == H) {
      c32 a = src[x], m = src[(N - x) & (N - 1)];
      v = r == 0 ? c32{0.5f * (a.x + m.x), 0.5f * (a.y - m.y)}
                 : c32{0.5f * (a.y + m.y), 0.5f * (m.x - a.x)};
    } else {
      v = src[r * RS + x];
    }
    dst[bin * binStride] = v;
  }
}

// ---- 3. C[bin][i][j] -> planes (i, j), cropped ----
template <int N>
__global__ __launch_bounds__(kT) void inverseBinMajor(const float2* Cs, int I, int Jp, PlaneSet out) {
  using C = BMCfg<N>;
  constexpr int H = C::H, T = C::T, SLOTS = C::SLOTS, RS = C::RS, PSZ = C::PSZ;
  __shared__ __align__(16) c32 lds[SLOTS * PSZ];
  const int t = threadIdx.x;
  const int s = t / T, l = t % T;
  const int j0 = blockIdx.x * SLOTS;
  const int i = blockIdx.y;

  const int sp = t % SLOTS, bq = t / SLOTS;
  {
    // gather: every load is issued before the first LDS store
    constexpr int PER = C::BINS / T;
    static_assert(C::BINS % T == 0, "bins divide evenly over the lane groups");
    c32* dstp = lds + sp * PSZ;
    const float2* src = Cs + (long)i * Jp + j0 + sp;
    const long binStride = (long)I * Jp;
    c32 in[PER];
    staticFor<PER>([&](auto uu) {
      constexpr int u = decltype(uu)::value;
      in[u] = src[(bq + T * u) * binStride];
    });
    staticFor<PER>([&](auto uu) {
      constexpr int u = decltype(uu)::value;
      const int bin = bq + T * u;
      dstp[(bin / N) * RS + bin % N] = in[u];
    });
  }
  __syncthreads();
  c32* plane = lds + s * PSZ;
  {  // pack rows 0 and H: Q = F0 + i*FH, real parts only at x = 0 (fbfft/FFT2D32.cuh:310-316)
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
  }
  __syncthreads();
  rowPassInPlace<N, false>(plane, l);
  __syncthreads();
  c32 z0[H], z1[H];
  columnPassInverse<N>(plane, l, z0, z1);
  const int j = j0 + s;
  if (j < out.K)  // out.K: number of valid output planes along j
    storeColumnsWindow<N>(out.base + (long)i * out.sRow + (long)j * out.sK, out.sy, out.sx, out.h,
                          out.w, 0, 0, l, z0, z1, 1.0f);
}

// ---- 2. batched complex GEMM, bin-major ----
constexpr int GI = 128;

struct GemmArgs {
  const float2* A;  // [bins][Kp][Ip]
  const float2* B;  // [bins][Kp][Jp]
  float2* C;        // [bins][I][Jp]
  int bins, I, Ip, Jp, Kp;
  int IT, JT;       // tiles per bin
  float invNorm;
};

template <int GJ, int GK>
__global__ __launch_bounds__(kT, 2) void binGemm(GemmArgs g) {
  constexpr int NA = GK * GI / 2 / kT;                 // float4 of A per lane per slice
  constexpr int NB = (GK * GJ / 2 + kT - 1) / kT;      // float4 of B per lane per slice
  constexpr int NQ = GJ / 32;  // 32-column MFMA sub-tiles per wave
  __shared__ __align__(16) float2 As[2][GK][GI];
  __shared__ __align__(16) float2 Bs[2][GK][GJ];
  const int t = threadIdx.x;
  const int lane = t % 64, w = t / 64;
  const int r = lane % 32, h = lane / 32;

  // consecutive logical ids on one XCD (workgroups are dealt round-robin to 8 XCDs)
  const int total = g.bins * g.IT * g.JT;
  const int per = (total + 7) / 8;
  const int logical = (blockIdx.x % 8) * per + blockIdx.x / 8;
  if (logical >= total) return;
  const int bin = logical / (g.IT * g.JT);
  const int rem = logical % (g.IT * g.JT);
  const int i0 = (rem / g.JT) * GI, j0 = (rem % g.JT) * GJ;

  const float2* Ab = g.A + (long)bin * g.Kp * g.Ip;
  const float2* Bb = g.B + (long)bin * g.Kp * g.Jp;

  floatx16 cre[NQ], cim[NQ];
#pragma unroll
  for (int q = 0; q < NQ; ++q)
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      cre[q][v] = 0.f;
      cim[q][v] = 0.f;
    }

  // slice loads: A 8 x 128 complex = 512 float4 (2 per lane), B 8 x 64 = 256 float4 (1 per lane)
  float4 ra[NA], rb[NB];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int u = 0; u < NA; ++u) {
      const int idx = t + kT * u;
      const int kk = idx / (GI / 2), ii = 2 * (idx % (GI / 2));
      ra[u] = float4{0.f, 0.f, 0.f, 0.f};
      if (k0 + kk < g.Kp && i0 + ii < g.Ip)
        ra[u] = *reinterpret_cast<const float4*>(Ab + (long)(k0 + kk) * g.Ip + i0 + ii);
    }
#pragma unroll
    for (int u = 0; u < NB; ++u) {
      const int idx = t + kT * u;
      const int kk = idx / (GJ / 2), jj = 2 * (idx % (GJ / 2));
      rb[u] = float4{0.f, 0.f, 0.f, 0.f};
      if (kk < GK && k0 + kk < g.Kp && j0 + jj < g.Jp)
        rb[u] = *reinterpret_cast<const float4*>(Bb + (long)(k0 + kk) * g.Jp + j0 + jj);
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int u = 0; u < NA; ++u) {
      const int idx = t + kT * u;
      *reinterpret_cast<float4*>(&As[buf][idx / (GI / 2)][2 * (idx % (GI / 2))]) = ra[u];
    }
#pragma unroll
    for (int u = 0; u < NB; ++u) {
      const int idx = t + kT * u;
      if (idx / (GJ / 2) < GK)
        *reinterpret_cast<float4*>(&Bs[buf][idx / (GJ / 2)][2 * (idx % (GJ / 2))]) = rb[u];
    }
  };

  fetch(0);
  stash(0);
  __syncthreads();
  const int slices = (g.Kp + GK - 1) / GK;
  for (int sl = 0; sl < slices; ++sl) {
    const int cur = sl & 1;
    if (sl + 1 < slices) fetch((sl + 1) * GK);
#pragma unroll
    for (int s2 = 0; s2 < GK / 2; ++s2) {
      const float2 a = As[cur][2 * s2 + h][32 * w + r];
      const float nar = -a.x;
#pragma unroll
      for (int q = 0; q < NQ; ++q) {
        const float2 b = Bs[cur][2 * s2 + h][32 * q + r];
        // a * conj(b): re = ar*br + ai*bi, im = ai*br - ar*bi
        cre[q] = __builtin_amdgcn_mfma_f32_32x32x2f32(a.x, b.x, cre[q], 0, 0, 0);
        cim[q] = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, b.x, cim[q], 0, 0, 0);
        cre[q] = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, b.y, cre[q], 0, 0, 0);
        cim[q] = __builtin_amdgcn_mfma_f32_32x32x2f32(nar, b.y, cim[q], 0, 0, 0);
      }
    }
    if (sl + 1 < slices) stash(cur ^ 1);
    __syncthreads();
  }

  // register v of lane (r, h) holds row 8*(v/4) + 4*h + v%4 and column r of a sub-tile
  float2* Cb = g.C + (long)bin * g.I * g.Jp;
#pragma unroll
  for (int q = 0; q < NQ; ++q) {
    const int j = j0 + 32 * q + r;
    if (j >= g.Jp) continue;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int i = i0 + 32 * w + 8 * (v / 4) + 4 * h + v % 4;
      if (i < g.I) Cb[(long)i * g.Jp + j] = float2{cre[q][v] * g.invNorm, cim[q][v] * g.invNorm};
    }
  }
}

inline int roundUp(int a, int b) { return (a + b - 1) / b * b; }

template <int N>
size_t workspaceFloat2(int B, int Cin, int Cout) {
  const int SL = BMCfg<N>::SLOTS, bins = BMCfg<N>::BINS;
  const int Ip = roundUp(B, SL), Jp = roundUp(Cout, SL), Kp = roundUp(Cin, 2);
  return (size_t)bins * ((size_t)Kp * Ip + (size_t)Kp * Jp + (size_t)B * Jp);
}

template <int N>
int runFprop(const PlaneSet& in, const PlaneSet& wt, const PlaneSet& out, int B, int Cin, int Cout,
             float2* ws, hipStream_t s) {
  using C = BMCfg<N>;
  const int SL = C::SLOTS, bins = C::BINS;
  const int Ip = roundUp(B, SL), Jp = roundUp(Cout, SL), Kp = roundUp(Cin, 2);
  float2* SA = ws;
  float2* SB = SA + (size_t)bins * Kp * Ip;
  float2* SC = SB + (size_t)bins * Kp * Jp;

  forwardBinMajor<N><<<dim3(Ip / SL, Kp), dim3(kT), 0, s>>>(in, SA, Ip, Kp);
  forwardBinMajor<N><<<dim3(Jp / SL, Kp), dim3(kT), 0, s>>>(wt, SB, Jp, Kp);
  GemmArgs g;
  g.A = SA;
  g.B = SB;
  g.C = SC;
  g.bins = bins;
  g.I = B;
  g.Ip = Ip;
  g.Jp = Jp;
  g.Kp = Kp;
  g.IT = ceilDiv(B, GI);
  g.invNorm = 1.0f / (float)(N * N);
  static const int gjEnv = getenv("FBFFT_GEMM_GJ") ? atoi(getenv("FBFFT_GEMM_GJ")) : 64;
  static const int gkEnv = getenv("FBFFT_GEMM_GK") ? atoi(getenv("FBFFT_GEMM_GK")) : 8;
  g.JT = ceilDiv(Jp, gjEnv == 32 ? 32 : 64);
  const dim3 grid(roundUp(bins * g.IT * g.JT, 8));
  if (gjEnv == 32 && gkEnv == 16) binGemm<32, 16><<<grid, dim3(kT), 0, s>>>(g);
  else if (gjEnv == 32) binGemm<32, 8><<<grid, dim3(kT), 0, s>>>(g);
  else if (gkEnv == 16) binGemm<64, 16><<<grid, dim3(kT), 0, s>>>(g);
  else if (gkEnv == 4) binGemm<64, 4><<<grid, dim3(kT), 0, s>>>(g);
  else binGemm<64, 8><<<grid, dim3(kT), 0, s>>>(g);
  inverseBinMajor<N><<<dim3(Jp / SL, B), dim3(kT), 0, s>>>(SC, B, Jp, out);
  return launchStatus();
}

}  // namespace

size_t convFpropWorkspaceBytes(int N, int B, int Cin, int Cout) {
  size_t n = N == 8 ? workspaceFloat2<8>(B, Cin, Cout)
                    : N == 16 ? workspaceFloat2<16>(B, Cin, Cout) : workspaceFloat2<32>(B, Cin, Cout);
  return n * sizeof(float2);
}

// input [B][Cin][H][W], weight [Cout][Cin][kH][kW], output [B][Cout][oH][oW]; strides in floats
int launchConvFprop(int N, float* in, const int* inStride, const int* inSize, float* wt,
                    const int* wtStride, const int* wtSize, float* out, const int* outStride,
                    const int* outSize, void* workspace, hipStream_t s) {
  const int B = inSize[0], Cin = inSize[1], Cout = wtSize[0];
  PlaneSet pin{in, inStride[0], inStride[1], inStride[2], inStride[3], inSize[2], inSize[3], B, Cin};
  PlaneSet pwt{wt, wtStride[0], wtStride[1], wtStride[2], wtStride[3], wtSize[2], wtSize[3], Cout, Cin};
  // for the output, "row" is the image and "k" the output plane
  PlaneSet pout{out, outStride[0], outStride[1], outStride[2], outStride[3], outSize[2], outSize[3],
                B, Cout};
  float2* ws = static_cast<float2*>(workspace);
  switch (N) {
    case 8: return runFprop<8>(pin, pwt, pout, B, Cin, Cout, ws, s);
    case 16: return runFprop<16>(pin, pwt, pout, B, Cin, Cout, ws, s);
    case 32: return runFprop<32>(pin, pwt, pout, B, Cin, Cout, ws, s);
  }
  return FBFFT_UNSUPPORTED_SIZE;
}

}  // namespace fbfft_amd
