// Fused tiled FFT convolution: FFT -> multiply-accumulate -> IFFT in one kernel
// with no device scratch (replaces updateOutputIteratedKernel*,
// updateGradInputIteratedKernel* and accGradParametersIteratedKernel*,
// fbfft/FFTIteratedConvolution.cuh:97-570, and the entry points at :624-755).
//
// All three passes are one scheme: planes "A_a" and "W_w" are transformed for
// each step of a reduction and acc[a][w] += A_a (x) W_w is accumulated per
// frequency bin, then every acc plane is inverse-transformed and cropped into
// its destination window.
//
//   pass             step       A_a               W_w               acc -> destination
//   updateOutput     cin        ins[t](n_a, c)    weight(f_w, c)    a * conj(w) -> outs[t](n_a, f_w) / N^2
//   updateGradInput  cout       outs[t](n_a, f)   weight(f, c_w)    a * w       -> ins[t](n_a, c_w)  / N^2
//   accGradParams    tile, n    ins[t](n, c_a)    outs[t](n, f_w)   a * conj(w) -> weight(f_w, c_a) * scale / N^2
//
// The reference gives every (batch, plane) pair its own lanes and recomputes
// both forward transforms for each of them.  Here a 256-lane workgroup shares
// BN + FO = 3/4 * (512/N) forward transforms per step among BN * FO products
// (4 x 8 for N = 32, 8 x 16 for N = 16, 16 x 32 for N = 8): spectra pass through
// LDS once, and each lane keeps 64 complex accumulators for its own frequency
// bins in VGPRs across the whole reduction.  Spectral rows 0 and N/2 stay packed
// as one complex row throughout (fbfft/FFTIteratedConvolution.cuh:161-186), so
// the inverse needs no re-packing.
#include "common.h"
#include "fft2d_core.h"
#include "fft_regs.h"

namespace fbfft_amd {
namespace {

constexpr int kThreads = 256;

struct ConvArgs {
  const fbfft_tile* ins;
  const fbfft_tile* outs;
  float* weight;
  int ws[4];  // weight strides (floats)
  int wn[4];  // weight sizes: Cout, Cin, kH, kW
  int batch;
  int numTiles;
  float scale;
};

struct PlaneRef {
  float* p;
  int sy, sx, h, w, padL, padU;
  bool valid;
};

__device__ __forceinline__ PlaneRef tilePlane(const fbfft_tile& t, int n, int c, int batch) {
  PlaneRef r;
  r.valid = n < batch && n < t.size[0] && c < t.size[1];
  r.p = t.data + (size_t)n * t.stride[0] + (size_t)c * t.stride[1];
  r.sy = t.stride[2];
  r.sx = t.stride[3];
  r.h = t.size[2];
  r.w = t.size[3];
  r.padL = t.padL;
  r.padU = t.padU;
  return r;
}

__device__ __forceinline__ PlaneRef weightPlane(const ConvArgs& a, int f, int c) {
  PlaneRef r;
  r.valid = f < a.wn[0] && c < a.wn[1];
  r.p = a.weight + (size_t)f * a.ws[0] + (size_t)c * a.ws[1];
  r.sy = a.ws[2];
  r.sx = a.ws[3];
  r.h = a.wn[2];
  r.w = a.wn[3];
  r.padL = 0;
  r.padU = 0;
  return r;
}

template <int N>
struct ConvCfg {
  static constexpr int H = N / 2;
  static constexpr int T = N / 2;                  // lanes per plane transform
  static constexpr int SLOTS = kThreads / T;       // concurrent plane transforms
  static constexpr int FO = SLOTS / 2;             // W planes per workgroup
  static constexpr int BN = FO / 2;                // A planes per workgroup
  static constexpr int RS = PlaneCfg<N>::RS;
  static constexpr int PSZ = H * RS;               // packed plane in LDS (complex)
  static constexpr int PB = H * N;                 // packed bins per plane
  static constexpr int GRP = (PB >= kThreads) ? 1 : kThreads / PB;   // lane groups sharing a bin set
  static constexpr int NBT = (PB >= kThreads) ? PB / kThreads : 1;   // bins per lane
  static constexpr int FQ = FO / GRP;              // W planes per lane
  static_assert(BN * FQ * NBT == 64, "64 complex accumulators per lane");
};

// a (x) w for the pass: a * conj(w) or a * w
template <bool CONJ>
__device__ __forceinline__ c32 prod(c32 a, c32 w) {
  return CONJ ? c32{a.x * w.x + a.y * w.y, a.y * w.x - a.x * w.y}
              : c32{a.x * w.x - a.y * w.y, a.x * w.y + a.y * w.x};
}

// split a packed row-0 value into its two real-row spectra
__device__ __forceinline__ void unpack0(c32 self, c32 other, c32* r0, c32* rN2) {
  *r0 = c32{0.5f * (self.x + other.x), 0.5f * (self.y - other.y)};
  *rN2 = c32{0.5f * (self.y + other.y), 0.5f * (other.x - self.x)};
}

template <int N, int PASS>
__global__ __launch_bounds__(kThreads) void iteratedConvKernel(ConvArgs a) {
  using C = ConvCfg<N>;
  constexpr int H = C::H, T = C::T, SLOTS = C::SLOTS, FO = C::FO, BN = C::BN, RS = C::RS,
                PSZ = C::PSZ, PB = C::PB, GRP = C::GRP, NBT = C::NBT, FQ = C::FQ;
  constexpr bool CONJ = (PASS != 1);
  __shared__ __align__(16) c32 lds[SLOTS * PSZ];

  const int t = threadIdx.x;
  const int s = t / T, l = t % T;
  const int gidx = (GRP > 1) ? t / PB : 0;
  const int bin0 = (GRP > 1) ? t % PB : t;

  const int tile = blockIdx.x;        // passes 0, 1
  const int w0 = blockIdx.y * FO;     // first W plane (f for passes 0 and 2, c for pass 1)
  const int a0 = blockIdx.z * BN;     // first A plane (n for passes 0 and 1, c for pass 2)
  const int Cout = a.wn[0], Cin = a.wn[1];
  const int steps = PASS == 0 ? Cin : PASS == 1 ? Cout : a.numTiles * a.batch;

  c32 acc[BN][FQ][NBT];
#pragma unroll
  for (int i = 0; i < BN; ++i)
#pragma unroll
    for (int j = 0; j < FQ; ++j)
#pragma unroll
      for (int k = 0; k < NBT; ++k) acc[i][j][k] = c32{0.f, 0.f};

  c32* plane = lds + s * PSZ;
  for (int step = 0; step < steps; ++step) {
    // ---- forward transforms of this step's A and W planes ----
    if (s < BN + FO) {
      PlaneRef ref;
      if (PASS == 0) {
        ref = s < BN ? tilePlane(a.ins[tile], a0 + s, step, a.batch)
                     : weightPlane(a, w0 + s - BN, step);
      } else if (PASS == 1) {
        ref = s < BN ? tilePlane(a.outs[tile], a0 + s, step, a.batch)
                     : weightPlane(a, step, w0 + s - BN);
      } else {
        const int tl = step / a.batch, n = step % a.batch;
        ref = s < BN ? tilePlane(a.ins[tl], n, a0 + s, a.batch)
                     : tilePlane(a.outs[tl], n, w0 + s - BN, a.batch);
      }
      c32 z0[H], z1[H];
      if (ref.valid) {
        loadColumnsWindowPerLane<N>(ref.p, ref.sy, ref.sx, ref.h, ref.w, ref.padL, ref.padU, l, z0, z1);
      } else {
#pragma unroll
        for (int j = 0; j < H; ++j) z0[j] = z1[j] = c32{0.f, 0.f};
      }
      columnPassForward<N>(z0, z1, plane, l);
    }
    __syncthreads();
    if (s < BN + FO) rowPassInPlace<N, true>(plane, l);
    __syncthreads();

    // ---- acc[a][w] += A_a (x) W_w on this lane's bins ----
#pragma unroll
    for (int nb = 0; nb < NBT; ++nb) {
      const int bin = bin0 + kThreads * nb;
      const int r = bin / N, x = bin % N;
      const int o = r * RS + x;
      if (r != 0) {
        c32 wv[FQ];
#pragma unroll
        for (int q = 0; q < FQ; ++q) wv[q] = lds[(BN + gidx + GRP * q) * PSZ + o];
#pragma unroll
        for (int i = 0; i < BN; ++i) {
          const c32 av = lds[i * PSZ + o];
#pragma unroll
          for (int q = 0; q < FQ; ++q) {
            c32 p = prod<CONJ>(av, wv[q]);
            acc[i][q][nb].x += p.x;
            acc[i][q][nb].y += p.y;
          }
        }
      } else if (x != 0) {
        // packed row: two real-row spectra per value, multiplied separately and re-packed
        const int om = (N - x);
        c32 w0v[FQ], wHv[FQ];
#pragma unroll
        for (int q = 0; q < FQ; ++q) {
          const c32* wp = lds + (BN + gidx + GRP * q) * PSZ;
          unpack0(wp[x], wp[om], &w0v[q], &wHv[q]);
        }
#pragma unroll
        for (int i = 0; i < BN; ++i) {
          const c32* ap = lds + i * PSZ;
          c32 a0v, aHv;
          unpack0(ap[x], ap[om], &a0v, &aHv);
#pragma unroll
          for (int q = 0; q < FQ; ++q) {
            c32 p0 = prod<CONJ>(a0v, w0v[q]);
            c32 pH = prod<CONJ>(aHv, wHv[q]);
            acc[i][q][nb].x += p0.x - pH.y;  // p0 + i * pH
            acc[i][q][nb].y += p0.y + pH.x;
          }
        }
      } else {
        // x = 0: both halves are real (fbfft/FFTIteratedConvolution.cuh:176-180)
#pragma unroll
        for (int i = 0; i < BN; ++i) {
          const c32 av = lds[i * PSZ];
#pragma unroll
          for (int q = 0; q < FQ; ++q) {
            const c32 wv = lds[(BN + gidx + GRP * q) * PSZ];
            acc[i][q][nb].x += av.x * wv.x;
            acc[i][q][nb].y += av.y * wv.y;
          }
        }
      }
    }
    __syncthreads();
  }

  // ---- inverse transforms, 2 A planes x FO W planes per round ----
  const float norm = (PASS == 2 ? a.scale : 1.0f) / (float)(N * N);
#pragma unroll
  for (int rd = 0; rd < BN / 2; ++rd) {
#pragma unroll
    for (int ii = 0; ii < 2; ++ii)
#pragma unroll
      for (int q = 0; q < FQ; ++q)
#pragma unroll
        for (int nb = 0; nb < NBT; ++nb) {
          const int bin = bin0 + kThreads * nb;
          lds[(ii * FO + gidx + GRP * q) * PSZ + (bin / N) * RS + bin % N] = acc[2 * rd + ii][q][nb];
        }
    __syncthreads();
    rowPassInPlace<N, false>(plane, l);
    __syncthreads();
    {
      c32 z0[H], z1[H];
      columnPassInverse<N>(plane, l, z0, z1);
      const int ai = a0 + 2 * rd + s / FO;
      const int wi = w0 + s % FO;
      PlaneRef ref;
      if (PASS == 0)
        ref = tilePlane(a.outs[tile], ai, wi, a.batch);
      else if (PASS == 1)
        ref = tilePlane(a.ins[tile], ai, wi, a.batch);
      else
        ref = weightPlane(a, wi, ai);
      if (ref.valid)
        storeColumnsWindow<N>(ref.p, ref.sy, ref.sx, ref.h, ref.w, ref.padL, ref.padU, l, z0, z1,
                              norm);
    }
    __syncthreads();
  }
}

template <int N>
int launchPass(int pass, const ConvArgs& a, hipStream_t s) {
  using C = ConvCfg<N>;
  const int Cout = a.wn[0], Cin = a.wn[1];
  if (pass == FBFFT_UPDATE_OUTPUT) {
    dim3 grid(a.numTiles, ceilDiv(Cout, C::FO), ceilDiv(a.batch, C::BN));
    iteratedConvKernel<N, 0><<<grid, kThreads, 0, s>>>(a);
  } else if (pass == FBFFT_UPDATE_GRAD_INPUT) {
    dim3 grid(a.numTiles, ceilDiv(Cin, C::FO), ceilDiv(a.batch, C::BN));
    iteratedConvKernel<N, 1><<<grid, kThreads, 0, s>>>(a);
  } else {
    dim3 grid(1, ceilDiv(Cout, C::FO), ceilDiv(Cin, C::BN));
    iteratedConvKernel<N, 2><<<grid, kThreads, 0, s>>>(a);
  }
  return launchStatus();
}

}  // namespace

// returns 1 launched, 0 nothing matched, -FBFFT_HIP_ERROR on launch failure
int launchIteratedConv(int N, const fbfft_tile* ins, const fbfft_tile* outs, float* weight,
                       const int* wStride, const int* wSize, int pass, float scale, int batch,
                       size_t numTiles, hipStream_t s) {
  if (!(N == 8 || N == 16 || N == 32)) return 0;
  if (pass < 0 || pass > 2) return 0;
  ConvArgs a;
  a.ins = ins;
  a.outs = outs;
  a.weight = weight;
  for (int d = 0; d < 4; ++d) {
    a.ws[d] = wStride[d];
    a.wn[d] = wSize[d];
  }
  a.batch = batch;
  a.numTiles = (int)numTiles;
  a.scale = scale;
  if (batch <= 0 || numTiles == 0 || wSize[0] <= 0 || wSize[1] <= 0) return 1;  // nothing to do
  int rc = N == 8 ? launchPass<8>(pass, a, s) : N == 16 ? launchPass<16>(pass, a, s)
                                                        : launchPass<32>(pass, a, s);
  return rc == FBFFT_SUCCESS ? 1 : -rc;
}

}  // namespace fbfft_amd
