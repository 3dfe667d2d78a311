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
// updateOutput and updateGradInput run one workgroup per (tile, A group, W group).
// accGradParameters reduces over all tiles and images; its reduction is also cut
// into ranges that separate workgroups accumulate and add atomically into the
// zeroed weight gradient, so that the chip is filled.
//
// The reference gives every (batch, plane) pair its own lanes and recomputes
// both forward transforms for each of them.  Here a 512-lane workgroup owns
// BN x FO products (8 x 8 for N = 32, 16 x 16 for N = 16, 32 x 32 for N = 8) and
// takes two reduction steps per iteration: its 1024/N plane slots hold the BN + FO
// forward transforms of both steps, so every lane transforms in every iteration
// and 2 (BN + FO) transforms feed 2 BN FO products (one transform per 4, 8, 16
// products).  Spectra pass through LDS once, and each lane keeps 64 complex
// accumulators for its own frequency bins in VGPRs across the whole reduction.
// Spectral rows 0 and N/2 travel packed as one complex row through the transforms;
// the accumulators hold them apart.
#include "common.h"

#include <algorithm>
#include "fft2d_core.h"
#include "fft_regs.h"

namespace fbfft_amd {
namespace {

constexpr int kThreads = 512;

struct ConvArgs {
  const fbfft_tile* ins;
  const fbfft_tile* outs;
  float* weight;
  int ws[4];  // weight strides (floats)
  int wn[4];  // weight sizes: Cout, Cin, kH, kW
  int batch;
  int numTiles;
  int splits;  // accGradParameters: workgroups along x sharing one reduction
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
  // the plane pointer comes out of a descriptor in memory: say that it is device memory,
  // or every access through it is a flat instruction
  typedef __attribute__((address_space(1))) float* GlobalPtr;
  r.p = (float*)(GlobalPtr)(t.data + (size_t)n * t.stride[0] + (size_t)c * t.stride[1]);
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
  static constexpr int SPI = 2;                    // reduction steps per iteration
  static constexpr int FO = SLOTS / (2 * SPI);     // W planes per workgroup
  static constexpr int BN = FO;                    // A planes per workgroup
  static constexpr int RA = SLOTS / FO;            // A planes per round of inverse transforms
  static constexpr int RS = PlaneCfg<N>::RS;
  static constexpr int PSZ = H * RS;               // packed plane in LDS (complex)
  static constexpr int PB = H * N;                 // packed bins per plane
  static constexpr int GRP = (PB >= kThreads) ? 1 : kThreads / PB;   // lane groups sharing a bin set
  static constexpr int NBT = (PB >= kThreads) ? PB / kThreads : 1;   // bins per lane
  static constexpr int FQ = FO / GRP;              // W planes per lane
  static_assert(BN * FQ * NBT == 64, "64 complex accumulators per lane");
};

// acc += a (x) w for the pass: a * conj(w) or a * w.  Four chained multiply-adds: formed
// as a product that is then added, it is six instructions (multiply, multiply-add and
// add per component - the compiler may not reassociate the sum), and this kernel is
// bound by the vector instructions it issues.
template <bool CONJ>
__device__ __forceinline__ void accumulate(c32& acc, c32 a, c32 w) {
  acc.x = __builtin_fmaf(a.x, w.x, acc.x);
  acc.x = __builtin_fmaf(CONJ ? a.y : -a.y, w.y, acc.x);
  acc.y = __builtin_fmaf(a.y, w.x, acc.y);
  acc.y = __builtin_fmaf(CONJ ? -a.x : a.x, w.y, acc.y);
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
                PSZ = C::PSZ, PB = C::PB, GRP = C::GRP, NBT = C::NBT, FQ = C::FQ, SPI = C::SPI,
                RA = C::RA;
  static_assert((BN + FO) * SPI == SLOTS && BN % RA == 0, "slot layout");
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
  // accGradParameters reduces over every (tile, image) pair; that reduction is cut
  // into a.splits ranges along blockIdx.x whose results meet in an atomic add
  const int perSplit = PASS == 2 ? ((steps + a.splits - 1) / a.splits + SPI - 1) / SPI * SPI : steps;
  const int stepBegin = PASS == 2 ? (int)blockIdx.x * perSplit : 0;
  const int stepEnd = min(steps, stepBegin + perSplit);

  c32 acc[BN][FQ][NBT];
#pragma unroll
  for (int i = 0; i < BN; ++i)
#pragma unroll
    for (int j = 0; j < FQ; ++j)
#pragma unroll
      for (int k = 0; k < NBT; ++k) acc[i][j][k] = c32{0.f, 0.f};

  c32* plane = lds + s * PSZ;
  // slot s transforms plane sj of reduction step SPI * it + su
  const int su = s / (BN + FO), sj = s % (BN + FO);
  for (int it = stepBegin / SPI; it < (stepEnd + SPI - 1) / SPI; ++it) {
    // ---- forward transforms of this iteration's A and W planes ----
    {
      const int step = SPI * it + su;
      PlaneRef ref;
      if (PASS == 0) {
        ref = sj < BN ? tilePlane(a.ins[tile], a0 + sj, step, a.batch)
                      : weightPlane(a, w0 + sj - BN, step);
      } else if (PASS == 1) {
        ref = sj < BN ? tilePlane(a.outs[tile], a0 + sj, step, a.batch)
                      : weightPlane(a, step, w0 + sj - BN);
      } else {
        // past the last step the tile index is clamped; the plane is zeroed below
        const int tl = min(step / a.batch, a.numTiles - 1), n = step % a.batch;
        ref = sj < BN ? tilePlane(a.ins[tl], n, a0 + sj, a.batch)
                      : tilePlane(a.outs[tl], n, w0 + sj - BN, a.batch);
      }
      c32 z0[H], z1[H];
      if (ref.valid && step < stepEnd) {
        loadColumnsWindowPerLane<N>(ref.p, ref.sy, ref.sx, ref.h, ref.w, ref.padL, ref.padU, l, z0,
                                    z1);
      } else {
#pragma unroll
        for (int j = 0; j < H; ++j) z0[j] = z1[j] = c32{0.f, 0.f};
      }
      columnPassForward<N>(z0, z1, plane, l);
    }
    __syncthreads();
    rowPassInPlace<N, true>(plane, l);
    __syncthreads();

    // ---- acc[a][w] += A_a (x) W_w on this lane's bins ----
    // Packed row 0 holds P[x] = F0[x] + i*FH[x], the Hermitian spectra of the two
    // real rows 0 and N/2.  Its lanes do not multiply packed values (that takes both
    // products in every lane, fbfft/FFTIteratedConvolution.cuh:161-186): lane x < N/2
    // accumulates the row-0 product at x and lane N/2 + x the row-N/2 product at x,
    // one complex product each like every other bin.  x = 0 carries the real values
    // at 0 and N/2 of its row as (re, im) and multiplies them separately.
#pragma unroll 1
    for (int u = 0; u < SPI; ++u) {
      const c32* ldsu = lds + u * (BN + FO) * PSZ;
#pragma unroll
      for (int nb = 0; nb < NBT; ++nb) {
        const int bin = bin0 + kThreads * nb;
        const int r = bin / N, x = bin % N;
        c32 wv[FQ];
        if (r != 0) {
          const int o = r * RS + x;
#pragma unroll
          for (int q = 0; q < FQ; ++q) wv[q] = ldsu[(BN + gidx + GRP * q) * PSZ + o];
#pragma unroll
          for (int i = 0; i < BN; ++i) {
            const c32 av = ldsu[i * PSZ + o];
#pragma unroll
            for (int q = 0; q < FQ; ++q) accumulate<CONJ>(acc[i][q][nb], av, wv[q]);
          }
        } else {
          // Row 0.  v = this lane's real-row spectrum value of a plane: the row-0 or
          // row-N/2 half of the packed pair (x, N - x), or for x = 0 the two real
          // values at 0 and N/2 as (re, im).  The real pair must be multiplied
          // component by component; written as the same four multiply-adds as a
          // complex product, with the first factor split in (re, 0) and (0, im) and
          // the second factor's components routed accordingly, so that all lanes of
          // the row run one instruction stream.
          const int xx = x & (H - 1);
          const bool second = x >= H, pair = xx == 0;
          const int i1 = xx, i2 = pair ? H : N - xx;
          auto value = [&](const c32* p) __attribute__((always_inline)) {
            const c32 self = p[i1], other = p[i2];
            c32 r0, rH;
            unpack0(self, other, &r0, &rH);
            const c32 ends = second ? c32{self.y, other.y} : c32{self.x, other.x};
            const c32 half = second ? rH : r0;
            return pair ? ends : half;
          };
          float w2x[FQ];
#pragma unroll
          for (int q = 0; q < FQ; ++q) {
            wv[q] = value(ldsu + (BN + gidx + GRP * q) * PSZ);
            w2x[q] = pair ? wv[q].y : wv[q].x;
          }
#pragma unroll
          for (int i = 0; i < BN; ++i) {
            const c32 av = value(ldsu + i * PSZ);
            const float a1y = pair ? 0.0f : av.y, a2x = pair ? 0.0f : av.x;
#pragma unroll
            for (int q = 0; q < FQ; ++q) {
              c32& to = acc[i][q][nb];
              to.x = __builtin_fmaf(av.x, wv[q].x, to.x);
              to.x = __builtin_fmaf(CONJ ? a1y : -a1y, wv[q].y, to.x);
              to.y = __builtin_fmaf(av.y, w2x[q], to.y);
              to.y = __builtin_fmaf(CONJ ? -a2x : a2x, wv[q].y, to.y);
            }
          }
        }
      }
    }
    __syncthreads();
  }

  // ---- inverse transforms, RA A planes x FO W planes per round ----
  const float norm = (PASS == 2 ? a.scale : 1.0f) / (float)(N * N);
#pragma unroll
  for (int rd = 0; rd < BN / RA; ++rd) {
    // Row-0 lanes park their value in the plane's padding (columns N, N+1 of row
    // x/2: N spare cells per plane) where the partner lane finds it.
#pragma unroll
    for (int ii = 0; ii < RA; ++ii)
#pragma unroll
      for (int q = 0; q < FQ; ++q)
#pragma unroll
        for (int nb = 0; nb < NBT; ++nb) {
          const int bin = bin0 + kThreads * nb;
          const int x = bin % N;
          const int o = bin < N ? (x / 2) * RS + N + x % 2 : (bin / N) * RS + x;
          lds[(ii * FO + gidx + GRP * q) * PSZ + o] = acc[RA * rd + ii][q][nb];
        }
    __syncthreads();
    // Row 0 back to its packed form Q[x] = S0[x] + i*SH[x], Q[N-x] = conj(S0[x]) +
    // i*conj(SH[x]): the lane holding S0[x] fetches SH[x] and writes Q[x], the lane
    // holding SH[x] fetches S0[x] and writes Q[N-x]; the two real pairs swap halves.
#pragma unroll
    for (int nb = 0; nb < NBT; ++nb) {
      const int bin = bin0 + kThreads * nb;
      if (bin < N) {
        const int x = bin, xx = x & (H - 1);
        const bool second = x >= H;
        const int px = second ? xx : H + xx;  // partner's x
        const int src = (px / 2) * RS + N + px % 2;
        const int dst = xx == 0 ? x : second ? N - xx : x;
#pragma unroll
        for (int ii = 0; ii < RA; ++ii)
#pragma unroll
          for (int q = 0; q < FQ; ++q) {
            c32* pl = lds + (ii * FO + gidx + GRP * q) * PSZ;
            const c32 mine = acc[RA * rd + ii][q][nb];
            const c32 other = pl[src];
            c32 v;
            if (xx == 0)
              v = second ? c32{other.y, mine.y} : c32{mine.x, other.x};
            else
              v = second ? c32{other.x + mine.y, mine.x - other.y}
                         : c32{mine.x - other.y, mine.y + other.x};
            pl[dst] = v;
          }
      }
    }
    __syncthreads();
    rowPassInPlace<N, false>(plane, l);
    __syncthreads();
    {
      c32 z0[H], z1[H];
      columnPassInverse<N>(plane, l, z0, z1);
      const int ai = a0 + RA * rd + s / FO;
      const int wi = w0 + s % FO;
      PlaneRef ref;
      if (PASS == 0)
        ref = tilePlane(a.outs[tile], ai, wi, a.batch);
      else if (PASS == 1)
        ref = tilePlane(a.ins[tile], ai, wi, a.batch);
      else
        ref = weightPlane(a, wi, ai);
      if (ref.valid) {
        if (PASS == 2 && a.splits > 1)
          storeColumnsWindow<N, true, true>(ref.p, ref.sy, ref.sx, ref.h, ref.w, ref.padL, ref.padU,
                                            l, z0, z1, norm);
        else
          storeColumnsWindow<N>(ref.p, ref.sy, ref.sx, ref.h, ref.w, ref.padL, ref.padU, l, z0, z1,
                                norm);
      }
    }
    __syncthreads();
  }
}

// weight[f][c][y][x] = 0 through its strides (a fill kernel, so that the call
// stays capturable in a graph)
__global__ void zeroWeight(ConvArgs a) {
  const long total = (long)a.wn[0] * a.wn[1] * a.wn[2] * a.wn[3];
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
    long r = i;
    const int x = r % a.wn[3];
    r /= a.wn[3];
    const int y = r % a.wn[2];
    r /= a.wn[2];
    const int c = r % a.wn[1];
    const int f = r / a.wn[1];
    a.weight[(long)f * a.ws[0] + (long)c * a.ws[1] + (long)y * a.ws[2] + (long)x * a.ws[3]] = 0.0f;
  }
}

template <int N>
int launchPass(int pass, const ConvArgs& a, bool deterministic, hipStream_t s) {
  using C = ConvCfg<N>;
  const int Cout = a.wn[0], Cin = a.wn[1];
  if (pass == FBFFT_UPDATE_OUTPUT) {
    dim3 grid(a.numTiles, ceilDiv(Cout, C::FO), ceilDiv(a.batch, C::BN));
    iteratedConvKernel<N, 0><<<grid, kThreads, 0, s>>>(a);
  } else if (pass == FBFFT_UPDATE_GRAD_INPUT) {
    dim3 grid(a.numTiles, ceilDiv(Cin, C::FO), ceilDiv(a.batch, C::BN));
    iteratedConvKernel<N, 1><<<grid, kThreads, 0, s>>>(a);
  } else {
    // The reference runs one block per group of planes over the whole reduction
    // (fbfft/FFTIteratedConvolution.cuh:600-613).  With 256 CUs that leaves most of the
    // chip idle, so the reduction is also split along x until there are about two
    // workgroups per CU; the partial gradients are then added atomically into a
    // zeroed weight tensor (summation order, hence the last bits, vary from run to
    // run).  A single split stores directly.
    ConvArgs b = a;
    const int groups = ceilDiv(Cout, C::FO) * ceilDiv(Cin, C::BN);
    const int steps = a.numTiles * a.batch;
    // deterministic: the reference's schedule, one workgroup per plane group over the
    // whole reduction in a fixed order, no atomics (and most of the chip idle)
    b.splits = deterministic
                   ? 1
                   : std::max(1, std::min(ceilDiv(512, groups), ceilDiv(steps, 2 * C::SPI)));
    if (b.splits > 1) {
      const long total = (long)a.wn[0] * a.wn[1] * a.wn[2] * a.wn[3];
      zeroWeight<<<dim3((unsigned)std::min<long>((total + 255) / 256, 4096)), 256, 0, s>>>(b);
    }
    dim3 grid(b.splits, ceilDiv(Cout, C::FO), ceilDiv(Cin, C::BN));
    iteratedConvKernel<N, 2><<<grid, kThreads, 0, s>>>(b);
  }
  return launchStatus();
}

}  // namespace

// returns 1 launched, 0 nothing matched, -FBFFT_HIP_ERROR on launch failure
int launchIteratedConv(int N, const fbfft_tile* ins, const fbfft_tile* outs, float* weight,
                       const int* wStride, const int* wSize, int pass, float scale, int batch,
                       size_t numTiles, bool deterministic, hipStream_t s) {
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
  a.splits = 1;
  a.scale = scale;
  if (batch <= 0 || numTiles == 0 || wSize[0] <= 0 || wSize[1] <= 0) return 1;  // nothing to do
  int rc = N == 8    ? launchPass<8>(pass, a, deterministic, s)
           : N == 16 ? launchPass<16>(pass, a, deterministic, s)
                     : launchPass<32>(pass, a, deterministic, s);
  return rc == FBFFT_SUCCESS ? 1 : -rc;
}

}  // namespace fbfft_amd
