// Per-frequency complex contraction on the fp32 matrix cores (replaces
// transposeMMTiledKernelUnrolled / ...Small / the generic fallback,
// MM-inl.cuh:34-506, and the dispatch at :515-814).
//
//   C[i][j][xy] = invNorm * ((accumulate ? C[i][j][xy] : 0) + sum_k opA[i][k][xy] * opB[k][j][xy])
//
// Operands keep the reference layout: complex, xy innermost and contiguous, so
// xy is the batch index of 'XY' independent small GEMMs and a coalesced global
// access is a run of consecutive bins of one (row, col) element.  Accumulators
// are needed for every bin of a run at once, which bounds the tile; a work item is
// a tile of C for 8 consecutive bins (64-byte runs; the other half of each line goes
// to the neighbouring workgroup on the same XCD).  Every path issues
// v_mfma_f32_32x32x2_f32, three real products per complex product
// (k1 = (Ar+Ai) Br, k2 = Ar (Bi-Br), k3 = Ai (Br+Bi); Cre = k1 - k3,
// Cim = k1 + k2), holds 192 accumulator registers per lane and sends C through LDS
// so that stores cover whole runs.  Only this contraction uses MFMA; it is the one
// dense product of the convolution path.
//
// Two kernels:
//  * the fast path (transposeMMDirectKernel, further down) for operands whose runs of
//    bin pairs are 16-byte aligned: 64 x 32 tiles, four waves of one bin pair each,
//    slices of k copied from HBM into LDS without passing through registers, two
//    workgroups per CU;
//  * the register path (transposeMMKernel) for everything else and for packed row 0:
//    a workgroup of 8 waves owns a 64 x 64 tile, wave w owning bin w.  Per 4-deep
//    slice of k it parks opA and opB in LDS split into real and imaginary planes
//    [bin][k][row] (conjugation folded into the sign of the imaginary plane, edges
//    zeroed), two buffers deep, while the slice after next is in flight in registers.
//
// Packed spectra (fbfft_transpose_mm_packed): operands [..][..][N/2][N] whose row 0
// holds P[x] = F0[x] + i FH[x], the spectra of the two real rows 0 and N/2 of an
// N x N transform (the Unpack = false format of fbfft/FFT2D32.cuh:421-427).  Rows
// 1 .. N/2-1 are plain bins and go through the register path.  Row 0 follows the
// product rule of fbfft/FFTIteratedConvolution.cuh:161-186: unpack both operands,
// multiply F0 with F0 and FH with FH, re-pack.  The PACKED0 variant of the kernel
// does that on the way into and out of LDS: a workgroup takes four x (0 < x < N/2)
// and its eight waves own the "virtual bins" F0[x] and FH[x], computed from P[x] and
// P[N-x] when a slice is parked; the epilogue combines C0[x] and CH[x] into P[x] and
// P[N-x].  x = 0 pairs with x = N/2: both hold two real values, which multiply
// component by component (no cross terms).
#include <utility>

#include "common.h"

namespace fbfft_amd {
namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int XB = 8;   // bins per work item: 64-byte runs of one (row, col) element
constexpr int KC = 4;   // k per slice
constexpr int CSTR = XB + 1;  // padded bin stride of the C staging buffer (complex)

// Shape of a work item.  WAVES waves share a TI x TJ tile of C for 8 consecutive
// bins; wave w owns bins w, w + WAVES, ...: (TI/32) x (TJ/32) MFMA sub-tiles x 3
// partial products x 16 registers for each of its bins - 192 accumulator registers
// for Wide (64 x 64, 8 waves of one bin), whose 512 lanes fill a CU.
template <int TI_, int TJ_, int WAVES_>
struct Geo {
  static constexpr int TI = TI_, TJ = TJ_, WAVES = WAVES_, THREADS = 64 * WAVES_;
  static constexpr int BW = XB / WAVES;  // bins per wave
  static constexpr int SI = TI / 32, SJ = TJ / 32;
  // bin stride of an LDS plane (dwords): the 4 bin pairs a half-wave writes land 8
  // banks apart
  static constexpr int XSA = KC * TI + 4, XSB = KC * TJ + 4;
  static constexpr int PLANE_A = XB * XSA, PLANE_B = XB * XSB;  // one of Ar, Ai / Br, Bi
  static constexpr int BUF = 2 * PLANE_A + 2 * PLANE_B;         // Ar, Ai, Br, Bi of one slice
  // C leaves in chunks of CR rows of the tile
  static constexpr int CR = 512 / TJ;
  static constexpr int STAGE_FLOATS = CR * TJ * CSTR * 2;
  static constexpr int LDS_FLOATS = (2 * BUF > STAGE_FLOATS) ? 2 * BUF : STAGE_FLOATS;
  static_assert(CR % 8 == 0 && 32 % CR == 0 && XB % WAVES == 0, "shape");
};
using Wide = Geo<64, 64, 8>;

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

// One slice of one operand: ROWS rows x KC k x 8 bins, fetched by THREADS lanes.  Lane
// t fetches bins 2p, 2p+1 (p = t % 4) of row (t/4) % ROWS at k = (t/4)/ROWS + KSTEP u:
// within a wave 16 consecutive rows, 64 bytes each.
template <int ROWS, int THREADS>
struct Fetch {
  static constexpr int KSTEP = THREADS / 4 / ROWS;  // k covered by one round of loads
  static constexpr int NF = KC / KSTEP;
  static_assert(KSTEP >= 1 && KC % KSTEP == 0, "shape");
  float4 v[NF];
};

// bin that shares its two spectra with bin x of a packed row 0
__device__ __forceinline__ int packedPartner(int x, int N) { return x == 0 ? N / 2 : N - x; }

// compile-time loop: f(std::integral_constant<int, 0>{}) ... f(<N-1>)
template <typename F, int... Is>
__device__ __forceinline__ void unrolledImpl(F&& f, std::integer_sequence<int, Is...>) {
  (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void unrolled(F&& f) {
  unrolledImpl(static_cast<F&&>(f), std::make_integer_sequence<int, N>{});
}

// What a lane needs to fetch and park its share of the slices of one operand.
// Every load is issued unconditionally at an address clamped into the operand; the
// values outside it are zeroed only when the slice is parked in LDS one iteration
// later, so nothing waits for a load between its issue and the products of the
// current slice.  VEC4 additionally needs XY even (a bin pair never straddles the end).
// PACKED0: XY is the length N of packed row 0, x0 a multiple of 4 below N/2; lane
// t fetches P[x] and P[partner(x)] for x = x0 + t % 4.
template <bool VEC4, bool PACKED0, int ROWS, int THREADS, int XS>
struct OperandLane {
  using F = Fetch<ROWS, THREADS>;
  const float* src0;  // the lane's row, at its first bin
  long kStride;
  long off2;     // PACKED0: floats from P[x] to P[partner]; else to the pair's second bin
  int kk0;       // the lane's k within a round of loads
  int K;
  int slot;      // dword offset of (k = kk0, row) in a bin of the LDS planes
  int p;
  float sign;
  bool okRow, okX1, ends;

  __device__ __forceinline__ OperandLane(const float* base, long rowStride, long kStride_,
                                         float sign_, int rows, int row0, int K_, int XY, int x0,
                                         int t)
      : kStride(kStride_), K(K_), sign(sign_) {
    p = t % 4;
    const int e = t / 4;
    const int row = row0 + e % ROWS;
    kk0 = e / ROWS;
    slot = kk0 * ROWS + e % ROWS;
    const float* rowBase = base + (long)min(row, rows - 1) * rowStride;
    if constexpr (PACKED0) {
      const int x = x0 + p;
      src0 = rowBase + 2L * x;
      off2 = 2L * (packedPartner(x, XY) - x);
      okRow = row < rows;
      okX1 = true;
      ends = x == 0;
    } else {
      const int x = x0 + 2 * p;
      src0 = rowBase + 2L * min(x, XY - (VEC4 ? 2 : 1));
      off2 = x + 1 < XY ? 2 : 0;
      okRow = row < rows && x < XY;
      okX1 = x + 1 < XY;
      ends = false;
    }
  }

  // load u of the slice that starts at k0
  __device__ __forceinline__ void fetch(F& f, int u, int k0) const {
    const int k = k0 + kk0 + F::KSTEP * u;
    const float* src = src0 + (long)min(k, K - 1) * kStride;
    if constexpr (VEC4 && !PACKED0) {
      f.v[u] = *reinterpret_cast<const float4*>(src);
    } else {
      const float2 a = *reinterpret_cast<const float2*>(src);
      const float2 b = *reinterpret_cast<const float2*>(src + off2);
      f.v[u] = float4{a.x, a.y, b.x, b.y};
    }
  }

  // parks load u of the slice that starts at k0 in the planes [bin][k][row] (bin
  // stride XS), zeroing what lies outside the operand
  __device__ __forceinline__ void stash(float* re, float* im, const F& f, int u, int k0) const {
    const int kk = kk0 + F::KSTEP * u;
    const int o = slot + F::KSTEP * u * ROWS;
    const bool ok = okRow && k0 + kk < K;
    const float4 v = f.v[u];
    if constexpr (PACKED0) {
      // virtual bin p: F0[x], virtual bin 4 + p: FH[x] from P[x] = (v.x, v.y) and
      // P[partner] = (v.z, v.w); for x = 0 the two bins hold the real pairs
      // (F0[0], F0[N/2]) and (FH[0], FH[N/2]), which conjugation leaves alone
      const float r0 = ends ? v.x : 0.5f * (v.x + v.z);
      const float i0 = ends ? v.z : sign * 0.5f * (v.y - v.w);
      const float rH = ends ? v.y : 0.5f * (v.y + v.w);
      const float iH = ends ? v.w : sign * 0.5f * (v.z - v.x);
      re[p * XS + o] = ok ? r0 : 0.f;
      im[p * XS + o] = ok ? i0 : 0.f;
      re[(4 + p) * XS + o] = ok ? rH : 0.f;
      im[(4 + p) * XS + o] = ok ? iH : 0.f;
    } else {
      re[(2 * p) * XS + o] = ok ? v.x : 0.f;
      im[(2 * p) * XS + o] = ok ? sign * v.y : 0.f;
      re[(2 * p + 1) * XS + o] = ok && okX1 ? v.z : 0.f;
      im[(2 * p + 1) * XS + o] = ok && okX1 ? sign * v.w : 0.f;
    }
  }
};

// one workgroup's share: work item `logical` of a (PACKED0: of the packed row 0 of a)
template <typename G, bool VEC4, bool PACKED0>
__device__ __forceinline__ void transposeMMBody(const MMArgs& a, int logical, float* lds) {
  constexpr int TI = G::TI, TJ = G::TJ, SI = G::SI, SJ = G::SJ, BW = G::BW, WAVES = G::WAVES;
  constexpr int THREADS = G::THREADS, XSA = G::XSA, XSB = G::XSB, BUF = G::BUF, CR = G::CR;
  // PACKED0 pairs virtual bins b and b + 4: both must sit in one wave or in waves that
  // agree on `ends`
  static_assert(WAVES == 4 || WAVES == 8, "shape");
  const int t = threadIdx.x;
  const int lane = t % 64, w = t / 64;
  const int tilesJ = (a.J + TJ - 1) / TJ, tilesI = (a.I + TI - 1) / TI;
  const int x0 = (logical / (tilesI * tilesJ)) * (PACKED0 ? XB / 2 : XB);
  const int rem = logical % (tilesI * tilesJ);
  // PACKED0: the waves holding the real pairs of x = 0 (virtual bins 0 and 4) multiply
  // component by component
  const bool ends = PACKED0 && x0 == 0 && w % 4 == 0;
  const float cross = ends ? 0.f : 1.f;
  const int j0 = (rem % tilesJ) * TJ;
  const int i0 = (rem / tilesJ) * TI;

  // sub-tile (si, sj): rows 32*si.., columns 32*sj...  Three real products per complex
  // product: with a = ar + i ai, b = br + i bi (conjugation already in the sign of
  // the imaginary planes), a b = (k1 - k3) + i (k1 + k2) for
  //   k1 = (ar + ai) br,  k2 = ar (bi - br),  k3 = ai (br + bi).
  floatx16 k1[BW][SI][SJ], k2[BW][SI][SJ], k3[BW][SI][SJ];
#pragma unroll
  for (int b = 0; b < BW; ++b)
#pragma unroll
    for (int si = 0; si < SI; ++si)
#pragma unroll
      for (int sj = 0; sj < SJ; ++sj)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          k1[b][si][sj][r] = 0.f;
          k2[b][si][sj][r] = 0.f;
          k3[b][si][sj][r] = 0.f;
        }

  using FA = Fetch<TI, THREADS>;
  using FB = Fetch<TJ, THREADS>;
  const OperandLane<VEC4, PACKED0, TI, THREADS, XSA> la(a.A, a.aRow, a.aK, a.aSign, a.I, i0, a.K,
                                                        a.XY, x0, t);
  const OperandLane<VEC4, PACKED0, TJ, THREADS, XSB> lb(a.B, a.bCol, a.bK, a.bSign, a.J, j0, a.K,
                                                        a.XY, x0, t);
  FA fa;
  FB fb;
  // Side work of one slice, cut into pieces that the loop below deals out between its
  // matrix instructions: per load, parking what it brought of slice n+1 and issuing it
  // again for slice n+2 into the same registers - every load then has most of an
  // iteration to arrive.  The pieces run unconditionally (past the end of K they park
  // zeros and re-read the last k): without branches in the loop the compiler counts
  // the loads in flight exactly instead of waiting for all of them.
  constexpr int NS = FA::NF + FB::NF, NP = 2 * NS;
  auto piece = [&](auto idx, int buf, int k0) __attribute__((always_inline)) {
    constexpr int i = decltype(idx)::value, load = i / 2;
    float* base = lds + buf * BUF;
    if constexpr (i % 2 == 0) {
      if constexpr (load < FA::NF)
        la.stash(base, base + G::PLANE_A, fa, load, k0);
      else
        lb.stash(base + 2 * G::PLANE_A, base + 2 * G::PLANE_A + G::PLANE_B, fb, load - FA::NF, k0);
    } else {
      if constexpr (load < FA::NF)
        la.fetch(fa, load, k0 + KC);
      else
        lb.fetch(fb, load - FA::NF, k0 + KC);
    }
  };
  if (a.K > 0) {  // with K = 0 the operands may have no memory behind them
    unrolled<NS>([&](auto i) { piece(std::integral_constant<int, 2 * decltype(i)::value + 1>{}, 0, -KC); });
    unrolled<NP>([&](auto i) { piece(i, 0, 0); });
  }
  __syncthreads();

  // Two slice buffers, one barrier per slice.  A slice is NG groups of products (a
  // step of two k for one of the wave's bins), a group SI * SJ sub-tiles of three
  // matrix instructions.  After each sub-tile the wave does one share of the side
  // work, so that no wave - and above all not both waves of a SIMD at once, as
  // happens when the side work sits right behind the barrier - leaves the matrix
  // pipeline alone for long; the operands of the next group are read one group ahead.
  constexpr int NG = (KC / 2) * BW, NSUB = NG * SI * SJ;
  struct Ops {
    float ar[SI], ai[SI], br[SJ], bi[SJ];
  };
  // the lane supplies row/col lane%32 (+32 per further sub-tile) at k = 2s + lane/32
  const int oa = lane % 32 + TI * (lane / 32), ob = lane % 32 + TJ * (lane / 32);
  auto readOps = [&](auto gg, int buf) __attribute__((always_inline)) {
    constexpr int g = decltype(gg)::value, st = g / BW, b = g % BW;
    const float* Ar = lds + buf * BUF;
    const float* Ai = Ar + G::PLANE_A;
    const float* Br = Ar + 2 * G::PLANE_A;
    const float* Bi = Br + G::PLANE_B;
    const int bin = w + WAVES * b;
    const int pa = bin * XSA + oa + st * 2 * TI, pb = bin * XSB + ob + st * 2 * TJ;
    Ops o;
#pragma unroll
    for (int q = 0; q < SI; ++q) {
      o.ar[q] = Ar[pa + 32 * q];
      o.ai[q] = Ai[pa + 32 * q];
    }
#pragma unroll
    for (int q = 0; q < SJ; ++q) {
      o.br[q] = Br[pb + 32 * q];
      o.bi[q] = Bi[pb + 32 * q];
    }
    return o;
  };
  int cur = 0;
  for (int k0 = 0; k0 < a.K; k0 += KC, cur ^= 1) {
    Ops ops[2];
    ops[0] = readOps(std::integral_constant<int, 0>{}, cur);
    unrolled<NG>([&](auto gg) {
      constexpr int g = decltype(gg)::value, b = g % BW;
      if constexpr (g + 1 < NG) ops[(g + 1) % 2] = readOps(std::integral_constant<int, g + 1>{}, cur);
      const Ops& o = ops[g % 2];
      float as[SI], bd[SJ], bs[SJ];
      // real pairs (cross = 0): k1 = sum ar br and k3 = sum ai bi are the two results
#pragma unroll
      for (int q = 0; q < SI; ++q)
        as[q] = PACKED0 ? __builtin_fmaf(cross, o.ai[q], o.ar[q]) : o.ar[q] + o.ai[q];
#pragma unroll
      for (int q = 0; q < SJ; ++q) {
        bs[q] = PACKED0 ? __builtin_fmaf(cross, o.br[q], o.bi[q]) : o.br[q] + o.bi[q];
        bd[q] = o.bi[q] - o.br[q];
      }
      unrolled<SI * SJ>([&](auto ss) {
        constexpr int sub = decltype(ss)::value, si = sub / SJ, sj = sub % SJ;
        __builtin_amdgcn_sched_barrier(0);
        k1[b][si][sj] =
            __builtin_amdgcn_mfma_f32_32x32x2f32(as[si], o.br[sj], k1[b][si][sj], 0, 0, 0);
        k2[b][si][sj] =
            __builtin_amdgcn_mfma_f32_32x32x2f32(o.ar[si], bd[sj], k2[b][si][sj], 0, 0, 0);
        k3[b][si][sj] =
            __builtin_amdgcn_mfma_f32_32x32x2f32(o.ai[si], bs[sj], k3[b][si][sj], 0, 0, 0);
        constexpr int n = g * SI * SJ + sub;  // sub-tile of the slice
        constexpr int first = n * NP / NSUB, last = (n + 1) * NP / NSUB;
        unrolled<last - first>([&](auto ii) {
          constexpr int i = first + decltype(ii)::value;
          piece(std::integral_constant<int, i>{}, cur ^ 1, k0 + KC);
        });
      });
    });
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();  // slice k0 consumed by everybody, slice k0 + KC parked by everybody
  }

  // ---- epilogue: C leaves through LDS so that every store covers whole runs (the
  // 8 bins of one (i, j) element).  Register r of lane l holds row
  // 8*(r/4) + 4*(l/32) + r%4 and column l%32 of a sub-tile, so registers 4g..4g+3 of
  // all lanes form rows 8g..8g+7 of a sub-tile row; a chunk is CR rows x TJ columns.
  float2* stage = reinterpret_cast<float2*>(lds);  // [CR rows][TJ cols][CSTR] complex
  const int col = lane % 32, hh = lane / 32;
  constexpr int GROUPS = CR / 8;           // register groups of 8 rows per chunk
  constexpr int PASSES = CR * TJ * XB / THREADS;
#pragma unroll
  for (int si = 0; si < SI; ++si)
#pragma unroll
    for (int c = 0; c < 32 / CR; ++c) {
      __syncthreads();  // operand slices / previous chunk fully consumed
#pragma unroll
      for (int b = 0; b < BW; ++b)
#pragma unroll
        for (int sj = 0; sj < SJ; ++sj)
#pragma unroll
          for (int g = 0; g < GROUPS; ++g)
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
              const int r = 4 * (GROUPS * c + g) + rr;
              const float v1 = k1[b][si][sj][r], v2 = k2[b][si][sj][r], v3 = k3[b][si][sj][r];
              stage[((8 * g + 4 * hh + rr) * TJ + 32 * sj + col) * CSTR + w + WAVES * b] =
                  ends ? float2{v1, v3} : float2{v1 - v3, v1 + v2};
            }
      __syncthreads();
      // CR * TJ (row, col) elements x 8 bins: 8 lanes per element
      const int xl = t % 8;
#pragma unroll
      for (int pass = 0; pass < PASSES; ++pass) {
        const int e = t / 8 + (THREADS / 8) * pass;
        const int row = e / TJ, cc = e % TJ;
        const int i = i0 + 32 * si + CR * c + row, j = j0 + cc;
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

template <typename G>
inline int workItems(const MMArgs& a) {
  return a.chunks * ceilDiv(a.J, G::TJ) * ceilDiv(a.I, G::TI);
}

// Workgroups are dealt round-robin to the 8 XCDs, each with its own L2.  Every XCD
// gets a contiguous range of logical ids, ordered bin-chunk first, so that the tiles
// that re-read the same lines of A and B (and the two chunks that share a 128-byte
// line) meet in one L2.
__device__ __forceinline__ int logicalWorkItem(int total) {
  const int per = (total + 7) / 8;
  return (blockIdx.x % 8) * per + blockIdx.x / 8;
}

// Built for two waves per SIMD (256 registers a lane): one Wide workgroup per CU.
template <typename G, bool VEC4>
__global__ __launch_bounds__(G::THREADS) __attribute__((amdgpu_waves_per_eu(2, 2))) void transposeMMKernel(MMArgs a, int total) {
  __shared__ __align__(8) float lds[G::LDS_FLOATS];  // two slice buffers; later the C staging area
  const int logical = logicalWorkItem(total);
  if (logical < total) transposeMMBody<G, VEC4, false>(a, logical, lds);
}

// Packed spectra in one launch: work items [0, totalMain) are the plain bins of rows
// 1 .. N/2-1, the rest the chunks of packed row 0 - a handful of workgroups that would
// leave most of the chip idle in a launch of their own.
template <typename G, bool VEC4>
__global__ __launch_bounds__(G::THREADS) __attribute__((amdgpu_waves_per_eu(2, 2))) void transposeMMPackedKernel(MMArgs mainRows,
                                                                      int totalMain, MMArgs row0,
                                                                      int totalRow0) {
  __shared__ __align__(8) float lds[G::LDS_FLOATS];
  // every XCD takes its share of the (slower) row-0 items first, then its range of
  // plain items
  const int perRow0 = (totalRow0 + 7) / 8, perMain = (totalMain + 7) / 8;
  const int xcd = blockIdx.x % 8, slot = blockIdx.x / 8;
  if (slot < perRow0) {
    const int item = xcd * perRow0 + slot;
    if (item < totalRow0) transposeMMBody<G, false, true>(row0, item, lds);
  } else {
    const int item = xcd * perMain + slot - perRow0;
    if (slot - perRow0 < perMain && item < totalMain)
      transposeMMBody<G, VEC4, false>(mainRows, item, lds);
  }
}

// ---- fast path: operands and C 16-byte aligned in every run of bin pairs, XY even ----
//
// Half-size work items (64 x 32) whose slices go from HBM straight into LDS (global_load_lds,
// 16 bytes per lane): no staging registers, no parking instructions - the side work
// per slice shrinks from some hundred vector instructions to six loads and their
// addresses, and vector instructions do not hide under the matrix pipeline here (the
// loop above loses the time they take even when they are dealt out between the matrix
// instructions).  LDS holds what HBM holds: a lane's 16 bytes are the two complex
// values of a bin pair, so wave w owns bin pair w (bins 2w, 2w+1) on the whole
// 64 x 32 tile and conjugation becomes a sign folded into the sums of the
// three-product form.
//
// A wave instruction fills 1 KiB = 16 rows x 4 bin pairs of one k, lane 4r + c taking
// pair c ^ (r / 4) of row r: four neighbouring lanes read one 64-byte run, and the 16
// rows of one pair land in 16 different 16-byte bank groups, so the 16-byte operand
// reads (32 rows of one pair at two k) meet no bank conflicts.
constexpr int DTJ = 32, DTHREADS = 256;
// rows of C per staging chunk: 8, or 4 where the stages (which the staging areas
// share their memory with) are small
constexpr int directChunkRows(int DTI) { return DTI == 64 ? 8 : 4; }

// [k][group of 16 rows][slot]; A and B of a stage are separate LDS variables
template <int DTI>
struct DirectA {
  float4 v[KC][DTI / 16][64];
};
struct DirectB {
  float4 v[KC][DTJ / 16][64];
};
// stages 0 and 1 of A double as the staging areas of C
template <int DTI>
struct DirectA0 {
  float4 v[KC][DTI / 16][64];
  float4 pad[(directChunkRows(DTI) * DTJ * CSTR * sizeof(float2) - sizeof(DirectA<DTI>)) / sizeof(float4)];
};

__device__ __forceinline__ int directSlot(int row16, int pair) { return 4 * row16 + (pair ^ (row16 / 4)); }

// A wave-uniform address pinned in scalar registers, and a lane's 32-bit offset kept
// apart from it up to the memory instruction: the empty statements keep the compiler
// from folding the two into a 64-bit vector addition per access, so that "scalar base +
// lane offset" reaches the instruction as its two operands.
template <class T>
__device__ __forceinline__ T* scalarBase(T* p) {
  asm volatile("" : "+s"(p));
  return p;
}
__device__ __forceinline__ unsigned laneOffset(unsigned& o) {
  asm volatile("" : "+v"(o));  // in place: the register is the same before and after, no copy
  return o;
}

__device__ __forceinline__ void loadToLds(const float* src, float4* ldsWaveBase) {
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                   (__attribute__((address_space(3))) void*)ldsWaveBase, 16, 0, 0);
}

// DTI: rows of the tile, 64, or 32 (one sub-tile per bin: 96 accumulator registers,
// three workgroups per CU, C staged in chunks of four rows)
template <int DTI>
__device__ __forceinline__ void transposeMMDirectBody(const MMArgs& a, int logical) {
  constexpr int SI = DTI / 32, DCR = directChunkRows(DTI);
  constexpr int DLOADS = DTI / 16 + DTJ / 16;  // global->LDS instructions per wave and slice
  // Six separate variables, not arrays of stages: the compiler tracks pending
  // global->LDS loads per LDS variable (and only for accesses that start at a
  // variable's first byte plus a run-time offset), so reading one stage does not wait
  // for the loads still in flight into the other two.
  __shared__ __align__(16) DirectA0<DTI> stageA0, stageA1;
  __shared__ __align__(16) DirectA<DTI> stageA2;
  __shared__ __align__(16) DirectB stageB0, stageB1, stageB2;
  const int t = threadIdx.x;
  const int lane = t % 64, w = __builtin_amdgcn_readfirstlane(t / 64);
  const int tilesJ = ceilDiv(a.J, DTJ), tilesI = ceilDiv(a.I, DTI);
  const int x0 = (logical / (tilesI * tilesJ)) * XB;
  const int rem = logical % (tilesI * tilesJ);
  const int j0 = (rem % tilesJ) * DTJ;
  const int i0 = (rem / tilesJ) * DTI;

  // loader role: wave w brings k-row w of every slice.  An address is a scalar base
  // (tile and k) plus a lane's byte offset within the tile, which never changes;
  // tiles whose rows lie too far apart for 32 bits are left to the other kernel by
  // the launcher.
  unsigned laneA[DTI / 16], laneB[DTJ / 16];
  {
    const int r = lane / 4, pair = (lane % 4) ^ (r / 4);
    const long xoff = 2L * (min(x0 + 2 * pair, a.XY - 2) - x0);
#pragma unroll
    for (int g = 0; g < DTI / 16; ++g)
      laneA[g] = (unsigned)(((long)(min(i0 + 16 * g + r, a.I - 1) - i0) * a.aRow + xoff) * (long)sizeof(float));
#pragma unroll
    for (int g = 0; g < DTJ / 16; ++g)
      laneB[g] = (unsigned)(((long)(min(j0 + 16 * g + r, a.J - 1) - j0) * a.bCol + xoff) * (long)sizeof(float));
  }
  const char* const tileA = (const char*)(a.A + (long)i0 * a.aRow + 2L * x0);
  const char* const tileB = (const char*)(a.B + (long)j0 * a.bCol + 2L * x0);
  const int slices = ceilDiv(a.K, KC);
  auto issue = [&](auto& stA, auto& stB, int sl) __attribute__((always_inline)) {
    const int k = min(sl * KC + w, a.K - 1);  // past the end: the last k again, zeroed before use
    const long offA = (long)k * a.aK * (long)sizeof(float), offB = (long)k * a.bK * (long)sizeof(float);
#pragma unroll
    for (int g = 0; g < DTI / 16; ++g)
      loadToLds((const float*)(scalarBase(tileA + offA) + laneOffset(laneA[g])), &stA.v[w][g][0]);
#pragma unroll
    for (int g = 0; g < DTJ / 16; ++g)
      loadToLds((const float*)(scalarBase(tileB + offB) + laneOffset(laneB[g])), &stB.v[w][g][0]);
  };

  // reader role: the lane supplies row/col lane%32 (+32 for the second sub-tile of A)
  // at k = 2s + lane/32, both bins of pair w in one 16-byte read
  const int r32 = lane % 32, kpar = lane / 32;
  const int slot = directSlot(r32 % 16, w), rg = r32 / 16;
  const int readA = (kpar * (DTI / 16) + rg) * 64 + slot, readB = (kpar * (DTJ / 16) + rg) * 64 + slot;
  const float sA = a.aSign, sB = a.bSign;

  // [bin of the pair][sub-tile of A]; a b = (k1 - sA k3) + i (k1 + k2) for
  //   k1 = (ar + sA ai) br,  k2 = ar (sB bi - br),  k3 = ai (br + sB bi)
  // (sA = +-1 is applied to k3 once, on the way out, not to every operand sum)
  floatx16 k1[2][SI], k2[2][SI], k3[2][SI];
#pragma unroll
  for (int h = 0; h < 2; ++h)
#pragma unroll
    for (int si = 0; si < SI; ++si)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        k1[h][si][r] = 0.f;
        k2[h][si][r] = 0.f;
        k3[h][si][r] = 0.f;
      }

  // One slice: wait for it, let everybody see it, request the slice two ahead into
  // the stage that was multiplied last time round, multiply.  Every step issues
  // exactly DLOADS loads (past the end it re-requests the last k into a stage nobody
  // reads), so "all but the newest DLOADS have landed" always means "slice sl has
  // landed".  The barrier is a bare s_barrier: no wave stores to these stages with
  // anything but the loads.
  auto step = [&](auto& curA, auto& curB, auto& refillA, auto& refillB, int sl)
                  __attribute__((always_inline)) {
    __builtin_amdgcn_s_waitcnt(0x0F70 | DLOADS);  // vmcnt(DLOADS)
    __builtin_amdgcn_s_barrier();
    if ((sl + 1) * KC > a.K) {
      // last, partial slice: the k beyond K hold copies of k = K-1
      for (int kz = a.K - sl * KC; kz < KC; ++kz) {
        if (t < 64 * (DTI / 16)) curA.v[kz][t / 64][t % 64] = float4{0.f, 0.f, 0.f, 0.f};
        if (t < 64 * (DTJ / 16)) curB.v[kz][t / 64][t % 64] = float4{0.f, 0.f, 0.f, 0.f};
      }
      __syncthreads();
    }
    issue(refillA, refillB, sl + 2);
    // left alone the compiler sinks the requests to the end of the step, which halves
    // the time they have to arrive
    __builtin_amdgcn_sched_barrier(0);
    const float4* flatA = &curA.v[0][0][0];
    const float4* flatB = &curB.v[0][0][0];
    float4 av[KC / 2][SI], bv[KC / 2];
#pragma unroll
    for (int s2 = 0; s2 < KC / 2; ++s2) {
      // one flat index per read: address chains of several steps lose the mark that
      // ties an access to its LDS variable
#pragma unroll
      for (int si = 0; si < SI; ++si)
        av[s2][si] = flatA[readA + (2 * s2) * (DTI / 16) * 64 + 2 * si * 64];
      bv[s2] = flatB[readB + (2 * s2) * (DTJ / 16) * 64];
    }
#pragma unroll
    for (int s2 = 0; s2 < KC / 2; ++s2) {
      const float br[2] = {bv[s2].x, bv[s2].z}, bi[2] = {bv[s2].y, bv[s2].w};
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const float bd = __builtin_fmaf(sB, bi[h], -br[h]);
        const float bs = __builtin_fmaf(sB, bi[h], br[h]);
#pragma unroll
        for (int si = 0; si < SI; ++si) {
          const float ar = h ? av[s2][si].z : av[s2][si].x, ai = h ? av[s2][si].w : av[s2][si].y;
          const float as = __builtin_fmaf(sA, ai, ar);
          k1[h][si] = __builtin_amdgcn_mfma_f32_32x32x2f32(as, br[h], k1[h][si], 0, 0, 0);
          k2[h][si] = __builtin_amdgcn_mfma_f32_32x32x2f32(ar, bd, k2[h][si], 0, 0, 0);
          k3[h][si] = __builtin_amdgcn_mfma_f32_32x32x2f32(ai, bs, k3[h][si], 0, 0, 0);
        }
      }
    }
  };

  if (slices > 0) {  // with K = 0 the operands may have no memory behind them
    issue(stageA0, stageB0, 0);
    issue(stageA1, stageB1, 1);
    int sl = 0;
    for (; sl + 3 <= slices; sl += 3) {
      step(stageA0, stageB0, stageA2, stageB2, sl);
      step(stageA1, stageB1, stageA0, stageB0, sl + 1);
      step(stageA2, stageB2, stageA1, stageB1, sl + 2);
    }
    if (sl < slices) {
      step(stageA0, stageB0, stageA2, stageB2, sl);
      if (sl + 1 < slices) step(stageA1, stageB1, stageA0, stageB0, sl + 1);
    }
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): nothing may land in LDS from here on

  // ---- epilogue: C leaves through LDS (the memory of A's stages 0 and 1) so that a
  // lane stores the 16 bytes of a bin pair and four lanes a whole 64-byte run.
  // Register r of lane l holds row 8*(r/4) + 4*(l/32) + r%4 and column l%32 of a
  // sub-tile: registers 4c..4c+3 of all lanes are rows 8c..8c+7, one chunk.  Chunks
  // alternate between two staging areas: one barrier per chunk, the next chunk is
  // parked while this one is stored.
  float2* stg[2] = {reinterpret_cast<float2*>(&stageA0), reinterpret_cast<float2*>(&stageA1)};
  const int col = lane % 32, hh = lane / 32;
  // chunk n: rows 32 si + 8 c + 4 half .. of the tile; with four rows per chunk only
  // the lanes of one half hold them
  constexpr int CHUNKS = 32 / DCR * SI, PER8 = 8 / DCR;
  auto park = [&](auto nn) __attribute__((always_inline)) {
    constexpr int n = decltype(nn)::value, si = n / (4 * PER8), c = n / PER8 % 4, half = n % PER8;
    float2* st = stg[n % 2];  // [DCR rows][32 cols][CSTR] complex
    if (DCR == 8 || hh == half) {
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
          const float v1 = k1[h][si][4 * c + rr], v2 = k2[h][si][4 * c + rr],
                      v3 = k3[h][si][4 * c + rr];
          st[(((DCR == 8 ? 4 * hh : 0) + rr) * DTJ + col) * CSTR + 2 * w + h] =
              float2{__builtin_fmaf(-sA, v3, v1), v1 + v2};
        }
    }
  };
  const int q = t % 4;
  // A tile that lies inside C whole (all but the last row, column or bin group of
  // tiles): an element's address is a scalar base per chunk and pass plus the lane's
  // fixed 32-bit offset, no tests and no 64-bit vector arithmetic per store.
  constexpr int ROWS_PER_PASS = DTHREADS / 4 / DTJ;
  const bool whole = i0 + DTI <= a.I && j0 + DTJ <= a.J && x0 + XB <= a.XY &&
                     (ROWS_PER_PASS * a.cRow + DTJ * a.cCol + 2 * XB) * (long)sizeof(float) < (1L << 31) &&
                     a.cRow >= 0 && a.cCol >= 0;
  unsigned laneC =
      (unsigned)((t / 4 / DTJ) * a.cRow + (t / 4 % DTJ) * a.cCol + 4 * q) * (unsigned)sizeof(float);
  char* const tileC = (char*)(a.C + (long)i0 * a.cRow + (long)j0 * a.cCol + 2L * x0);
  auto store = [&](auto nn) __attribute__((always_inline)) {
    constexpr int n = decltype(nn)::value, si = n / (4 * PER8), c = n / PER8 % 4, half = n % PER8;
    const float2* st = stg[n % 2];
    if (whole) {
      auto put = [&](auto accumulating) __attribute__((always_inline)) {
#pragma unroll
        for (int pass = 0; pass < DCR * DTJ * 4 / DTHREADS; ++pass) {
          const int e = t / 4 + (DTHREADS / 4) * pass;
          const float2 c0 = st[e * CSTR + 2 * q], c1 = st[e * CSTR + 2 * q + 1];
          typedef float __attribute__((ext_vector_type(4))) Quad;  // (float4's assignment takes a generic `this`)
          auto* dst = (__attribute__((address_space(1))) Quad*)(
              scalarBase(tileC + (32 * si + 8 * c + 4 * half + ROWS_PER_PASS * pass) * a.cRow *
                                     (long)sizeof(float)) +
              laneOffset(laneC));
          Quad acc{c0.x, c0.y, c1.x, c1.y};
          if constexpr (decltype(accumulating)::value) acc += *dst;
          *dst = acc * a.invNorm;
        }
      };
      if (a.accumulate)
        put(std::true_type{});
      else
        put(std::false_type{});
      return;
    }
#pragma unroll
    for (int pass = 0; pass < DCR * DTJ * 4 / DTHREADS; ++pass) {
      const int e = t / 4 + (DTHREADS / 4) * pass;
      const int row = e / DTJ, cc = e % DTJ;
      const int i = i0 + 32 * si + 8 * c + 4 * half + row, j = j0 + cc, x = x0 + 2 * q;
      const float2 c0 = st[e * CSTR + 2 * q], c1 = st[e * CSTR + 2 * q + 1];
      float4 acc{c0.x, c0.y, c1.x, c1.y};
      if (i < a.I && j < a.J && x < a.XY) {
        float* dst = a.C + (long)i * a.cRow + (long)j * a.cCol + 2L * x;
        if (a.accumulate) {
          const float4 old = *reinterpret_cast<const float4*>(dst);
          acc.x += old.x;
          acc.y += old.y;
          acc.z += old.z;
          acc.w += old.w;
        }
        *reinterpret_cast<float4*>(dst) = float4{acc.x * a.invNorm, acc.y * a.invNorm,
                                                 acc.z * a.invNorm, acc.w * a.invNorm};
      }
    }
  };
  __syncthreads();  // the last slice is consumed by everybody
  park(std::integral_constant<int, 0>{});
  __syncthreads();
  unrolled<CHUNKS>([&](auto nn) {
    constexpr int n = decltype(nn)::value;
    if constexpr (n + 1 < CHUNKS) park(std::integral_constant<int, n + 1>{});
    store(nn);
    if constexpr (n + 1 < CHUNKS) __syncthreads();
  });
}

template <int DTI>
inline int directWorkItems(const MMArgs& a) {
  return a.chunks * ceilDiv(a.J, DTJ) * ceilDiv(a.I, DTI);
}

// two (64 rows) or three (32 rows) workgroups per CU: one's C leaves while the others
// multiply
template <int DTI>
__global__ __launch_bounds__(DTHREADS) __attribute__((amdgpu_waves_per_eu(DTI == 64 ? 2 : 3, DTI == 64 ? 2 : 3)))
void transposeMMDirectKernel(MMArgs a, int total) {
  const int logical = logicalWorkItem(total);
  if (logical < total) transposeMMDirectBody<DTI>(a, logical);
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

bool storesAsFloat4(const float* C, long c0, long c1) {
  return aligned(C, 16) && c0 % 4 == 0 && c1 % 4 == 0;
}


template <typename G>
int launchPlain(const MMArgs& m, bool vec4, hipStream_t s) {
  const int total = workItems<G>(m);
  dim3 grid((total + 7) / 8 * 8), block(G::THREADS);
  if (vec4)
    transposeMMKernel<G, true><<<grid, block, 0, s>>>(m, total);
  else
    transposeMMKernel<G, false><<<grid, block, 0, s>>>(m, total);
  return launchStatus();
}

template <typename G>
int launchPacked(const MMArgs& mainRows, const MMArgs& row0, bool vec4, hipStream_t s) {
  const int totalMain = workItems<G>(mainRows), totalRow0 = workItems<G>(row0);
  dim3 grid(((totalMain + 7) / 8 + (totalRow0 + 7) / 8) * 8), block(G::THREADS);
  if (vec4)
    transposeMMPackedKernel<G, true><<<grid, block, 0, s>>>(mainRows, totalMain, row0, totalRow0);
  else
    transposeMMPackedKernel<G, false><<<grid, block, 0, s>>>(mainRows, totalMain, row0, totalRow0);
  return launchStatus();
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
  const bool vec4 = movesAsFloat4(A, a0, a1, B, b0, b1, XY);
  // (the fast path keeps a lane's offset within its tile, up to 63 rows, in 32 bits)
  const bool rowsNear = m.aRow >= 0 && m.aRow < (1L << 24) && m.bCol >= 0 && m.bCol < (1L << 24);
  if (vec4 && rowsNear && storesAsFloat4(C, c0, c1)) {
    // Equal work items are dealt to the CUs in whole numbers: the launch lasts as
    // long as the fullest CU.  32-row tiles re-read B twice as often and pay more per
    // matrix instruction, so they are taken only where they even the load out
    // (configs[3]: 816 items of 64 rows are 3.19 per CU, four on the fullest - 72 us;
    // 1632 of 32 rows are 6.4, seven on the fullest - 68 us; at 2, 4 or 8 items of 64
    // rows per CU the larger tile wins by 3-9 %).
    const int cus = computeUnits();
    auto evenness = [&](int items) { return (double)items / cus / ceilDiv(items, cus); };
    const int items64 = directWorkItems<64>(m), items32 = directWorkItems<32>(m);
    if (evenness(items32) > evenness(items64) + 0.05) {
      transposeMMDirectKernel<32><<<dim3((items32 + 7) / 8 * 8), dim3(DTHREADS), 0, s>>>(m, items32);
    } else {
      transposeMMDirectKernel<64><<<dim3((items64 + 7) / 8 * 8), dim3(DTHREADS), 0, s>>>(m, items64);
    }
    return launchStatus();
  }
  return launchPlain<Wide>(m, vec4, s);
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
  const bool vec4 = movesAsFloat4(A + 2 * N, a0, a1, B + 2 * N, b0, b1, XY);
  return launchPacked<Wide>(mainRows, row0, vec4, s);
}

}  // namespace fbfft_amd
