// The three passes of an FFT convolution layer (valid cross-correlation forward,
// its gradient with respect to the input, its gradient with respect to the
// weights), each as three kernels that hand spectra to each other in a layout
// chosen for the matrix cores.
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
//   2. binGemmDirect:    C[bin][i][j] = sum_k A[bin][k][i] * conj(B[bin][k][j])
//      one workgroup = one bin x (128 x 64) or (64 x 64) tile; k-slices of A and B
//      are contiguous in HBM and are copied verbatim into LDS by global_load_lds;
//      4 waves of MFMA 32x32x2 sub-tiles, three real products per complex one;
//      counters show A + B fetched
//      from HBM exactly once (the tiles of a bin share an L2: workgroup ids are
//      remapped per XCD) and C written once with coalesced stores.
//      binGemmRegsWide / binGemmRegsSplitK: the same product without LDS for
//      products with a side of up to 32 (planGemm picks kernel, tiles and the
//      ranges a long reduction is cut into).
//   3. inverseBinMajor:  C[bin][i][j] -> planes, gathering runs of SLOTS
//      consecutive j per bin, inverse transform, crop on store.
//
// The planes of an operand are a PlaneSet: whole tensors, overlapping windows of
// images larger than the transform (the layer entry points), or the tile
// descriptors of FFTIteratedConvolution in device memory (fbfft_iterated_conv_ws).
//
// Spectral rows 0 and N/2 of a real plane are both Hermitian along kx, so their
// 2 N complex values carry N complex worth of information; they travel as N
// "virtual bins": v = x (0 < x < N/2) is row 0 at x, v = N/2 + x is row N/2 at x, and
// v = 0 / v = N/2 hold the four real values (row 0 at 0 and N/2) / (row N/2 at 0 and
// N/2) as (re, im) pairs.  The contraction is then a plain complex GEMM on N^2/2 bins;
// only the two bins of real pairs multiply component by component instead (the product
// rule of fbfft/FFTIteratedConvolution.cuh:161-186 with the unpacking done once, when
// the forward transform stores the spectrum).
//
// All three passes are the same product P[i][j] = sum_k X[i][k] * op(Y[j][k]) with
// the roles of MM-inl.cuh:188-196: forward (i, j, k) = (image, output plane, input
// plane), op = conj; input gradient (image, input plane, output plane), op =
// identity; weight gradient (input plane, output plane, image), op = conj.  The
// kernels always compute sum_k A * conj(B); the forward transforms store a
// spectrum conjugated where the pass needs it.
#include "common.h"
#include "fft2d_core.h"
#include "fft_regs.h"

#include <utility>

namespace fbfft_amd {
namespace {

constexpr int kT = 256;
// lanes of a transform workgroup: 16 planes of 32 x 32, so that a bin leaves or arrives as
// a 128-byte run (measured at configs[3] / configs[4]: 128 lanes, 64-byte runs, +10 % /
// +12 % per pass; 512 lanes, one workgroup per CU, +8 % / +6 %)
constexpr int kTF = 256;
typedef float floatx16 __attribute__((ext_vector_type(16)));

template <int N>
struct BMCfg {
  static constexpr int H = N / 2;
  static constexpr int T = N / 2;
  static constexpr int SLOTS = kTF / T;                // planes per workgroup
  static constexpr int RS = PlaneCfg<N>::RS;
  // plane stride in LDS (complex): 16-byte aligned, and 4 banks mod 32 so that the
  // transposed accesses (16 or more planes at the same bin) spread over the banks
  static constexpr int PSZ = (H + 1) * RS;
  static_assert((2 * PSZ) % 32 == 4 && PSZ % 2 == 0, "plane stride");
  static constexpr int BINS = H * N;      // N virtual bins of rows 0 and N/2, then rows 1 .. N/2-1
};

// A family of planes indexed by (row, k).  Plain: plane (row, k) is the h x w window at
// base + row*sRow + k*sK.  Tiled (images larger than the transform): one of the two
// indices is the composite (image, tileY, tileX), image-major; its stride is the
// image stride, h x w is the whole image, and tile (ty, tx) is the winH x winW
// window at (orgY + ty*stepY, orgX + tx*stepX) clipped to the image - rows and
// columns clipped off above / left become the plane's padU / padL, so the window
// keeps its place inside the FFT plane.  padU0 / padL0 shift every window further
// (where a cropped result sits inside the inverse transform's plane).  Described
// (FFTIteratedConvolution's interface, fbfft/FFTIteratedConvolution.cuh:71-88): one of
// the two indices is the composite (image, tile), image-major, and every tile is a
// descriptor in device memory - a [batch][planes][h][w] view with its own strides and
// pads; the other index is the plane within the view.
struct PlaneSet {
  float* base;
  long sRow, sK;
  int sy, sx, h, w;
  int R, K;         // valid rows / k
  int tiled;        // 0: plain, 1: row is the composite index, 2: k is
  int tilesY, tilesX, stepY, stepX, orgY, orgX, winH, winW;
  int padU0, padL0;
  const fbfft_tile* tiles;  // described sets: the descriptors
  int described;            // 0: no, 1: row is the composite (image, tile), 2: k is
  int numTiles;             // tiles per image
};

// Orders the LDS accesses of one wave: what its lanes wrote before is what its lanes
// read after.  The lanes that share a plane sit in one wave, and a wave's LDS
// instructions execute in order, so the passes over a plane need no workgroup barrier
// between them - only the compiler has to keep the accesses in program order.
__device__ __forceinline__ void planeSync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

struct PlaneWindow {
  float* p;
  int h, w, padL, padU;
  int sy, sx;
  bool valid;  // described sets: the view holds this image and plane and is not empty
};

// DESCRIBED is a compile-time fact (the kernels' PAIRS == 2 instantiations): carried as a
// run-time test it cost the tiled sets 2 % (configs[4]: 290 against 284 us).
template <bool DESCRIBED>
__device__ __forceinline__ PlaneWindow planeWindow(const PlaneSet& ps, int row, int k) {
  if constexpr (DESCRIBED) {
    const int comp = ps.described == 1 ? row : k, other = ps.described == 1 ? k : row;
    // image-major: consecutive composites are consecutive tiles of one image - in a
    // row-major tiling neighbours in memory, which is what 16 planes of a workgroup should
    // be (tile-major, 16 images of one tile: 345 instead of 296 us at configs[4])
    const fbfft_tile& d = ps.tiles[comp % ps.numTiles];
    const int n = comp / ps.numTiles;
    PlaneWindow win;
    win.valid = n < d.size[0] && other < d.size[1] && d.size[2] > 0 && d.size[3] > 0;
    // a plane the view does not hold takes the place of one it does, and loads nothing
    // (no row passes the window test, and with padU = 0 no batch of rows is asked for)
    typedef __attribute__((address_space(1))) float* GlobalPtr;
    win.p = (float*)(GlobalPtr)(d.data + (long)min(n, max(d.size[0] - 1, 0)) * d.stride[0] +
                                (long)min(other, max(d.size[1] - 1, 0)) * d.stride[1]);
    win.h = max(d.size[2], 0);
    win.w = max(d.size[3], 0);
    win.padU = win.valid ? d.padU : 0;
    win.padL = d.padL;
    win.sy = d.stride[2];
    win.sx = d.stride[3];
    return win;
  }
  if (ps.tiled == 0)
    return PlaneWindow{ps.base + (long)row * ps.sRow + (long)k * ps.sK, ps.h, ps.w, ps.padL0,
                       ps.padU0, ps.sy, ps.sx, true};
  const int comp = ps.tiled == 1 ? row : k, other = ps.tiled == 1 ? k : row;
  const long sImg = ps.tiled == 1 ? ps.sRow : ps.sK, sOther = ps.tiled == 1 ? ps.sK : ps.sRow;
  const int perImage = ps.tilesY * ps.tilesX;
  const int img = comp / perImage, t = comp % perImage;
  const int y0 = ps.orgY + (t / ps.tilesX) * ps.stepY, x0 = ps.orgX + (t % ps.tilesX) * ps.stepX;
  const int ya = max(y0, 0), xa = max(x0, 0);
  PlaneWindow win;
  win.p = ps.base + (long)img * sImg + (long)other * sOther + (long)ya * ps.sy + (long)xa * ps.sx;
  win.h = min(y0 + ps.winH, ps.h) - ya;
  win.w = min(x0 + ps.winW, ps.w) - xa;
  win.padU = ps.padU0 + ya - y0;
  win.padL = ps.padL0 + xa - x0;
  win.sy = ps.sy;
  win.sx = ps.sx;
  win.valid = true;
  return win;
}

// ---- 1. planes -> S[bin][k][row] ----
// One operand of the product: its planes, where its spectra go, and how many
// workgroups (row groups x Kp) transform it.
struct ForwardJob {
  PlaneSet ps;
  float2* S;
  int Rp, Kp;
  float imSign;
  int rowGroups;  // workgroups per k: Rp / SLOTS, or half of that (rounded up) when a
                  // workgroup takes two runs of rows
  int stream;     // spectra leave with nontemporal stores
};

// Both operands of a pass in one launch: workgroups [0, a.rowGroups * a.Kp) transform
// a's planes, the rest b's.  PAIRS_x: every plane of that set passes
// windowMovesAsPairs() (8-byte words per row).  GROUPS (1 or 2): runs of SLOTS
// consecutive rows per workgroup; with two, the second run's planes are requested as
// soon as the first run's columns have left the registers and fly under the first
// run's row pass and stores.
template <int N, int PAIRS, int GROUPS>
__device__ __forceinline__ void forwardBinMajorBody(const ForwardJob& job, int wg, c32* lds);

template <int N, int PAIRS_A, int PAIRS_B, int GROUPS>
__global__ __launch_bounds__(kTF) void forwardBinMajor(ForwardJob a, ForwardJob b) {
  __shared__ __align__(16) c32 lds[BMCfg<N>::SLOTS * BMCfg<N>::PSZ];
  const int nA = a.rowGroups * a.Kp;
  if ((int)blockIdx.x < nA)
    forwardBinMajorBody<N, PAIRS_A, GROUPS>(a, blockIdx.x, lds);
  else
    forwardBinMajorBody<N, PAIRS_B, GROUPS>(b, blockIdx.x - nA, lds);
}

template <int N, int PAIRS, int GROUPS>
__device__ __forceinline__ void forwardBinMajorBody(const ForwardJob& job, int wg, c32* lds) {
  using C = BMCfg<N>;
  constexpr int H = C::H, T = C::T, SLOTS = C::SLOTS, RS = C::RS, PSZ = C::PSZ;
  const PlaneSet& ps = job.ps;
  float2* S = job.S;
  const int Rp = job.Rp, Kp = job.Kp;
  const float imSign = job.imSign;
  const int t = threadIdx.x;
  const int s = t / T, l = t % T;
  const int k = wg / job.rowGroups;
  c32* plane = lds + s * PSZ;

  auto load = [&](int r0, c32 (&z0)[H], c32 (&z1)[H]) __attribute__((always_inline)) {
    // padding planes (row >= R, k >= K) take the window of an existing plane and load nothing
    const int row = r0 + s;
    const PlaneWindow win = planeWindow<PAIRS == 2>(ps, min(row, ps.R - 1), min(k, ps.K - 1));
    const bool present = row < ps.R && k < ps.K && win.valid;
    // 4-byte loads (odd widths or strides): the lane takes columns l and l + N/2, so that
    // a load instruction reads neighbouring floats (configs[3]: input gradient 108.0 ->
    // 101.6 us, weight gradient 108.0 -> 104.1 us; forward pass unchanged).  PAIRS = 2
    // (described sets: the windows are only known on the device) decides per plane
    // between 8-byte and 4-byte loads of columns 2l and 2l + 1.
    loadColumnsWindow<N, PAIRS, PAIRS == 0>(win.p, win.sy, win.sx, win.h, win.w, win.padL, win.padU,
                                            l, z0, z1, present);
  };
  // lanes: sp = t % SLOTS walks the run (consecutive rows), bq = t / SLOTS in [0, T)
  // walks bins: lane (sp, bq) stores columns x = bq and bq + T of every spectral row,
  // so LDS and HBM offsets are compile-time constants on top of one per-lane base.
  auto copyOutAs = [&](int r0, auto streamTag) __attribute__((always_inline)) {
    const int sp = t % SLOTS, bq = t / SLOTS;
    const c32* src = lds + sp * PSZ + bq;
    const long binStride = (long)Kp * Rp;
    float2* dst = S + (long)k * Rp + r0 + sp + bq * binStride;
    auto put = [&](int bin, c32 v) __attribute__((always_inline)) {
      if constexpr (decltype(streamTag)::value)
        streamStore(dst + bin * binStride, v);
      else
        dst[bin * binStride] = v;
    };
    // Packed row 0 holds P[x] = F0[x] + i FH[x]: F0[x] = (P[x] + conj P[N-x]) / 2,
    // FH[x] = (P[x] - conj P[N-x]) / 2i.  Lane bq stores virtual bins bq (F0) and
    // T + bq (FH); bq = 0 stores the real pairs (F0[0], F0[N/2]) and (FH[0], FH[N/2]),
    // which no conjugation touches.
    {
      const c32 a = src[0], m = lds[sp * PSZ + (bq == 0 ? H : N - bq)];
      c32 f0 = c32{0.5f * (a.x + m.x), 0.5f * (a.y - m.y) * imSign};
      c32 fh = c32{0.5f * (a.y + m.y), 0.5f * (m.x - a.x) * imSign};
      if (bq == 0) {
        f0 = c32{a.x, m.x};
        fh = c32{a.y, m.y};
      }
      put(0, f0);
      put(T, fh);
    }
    staticFor<H - 1>([&](auto rr) {
      constexpr int r = decltype(rr)::value + 1;
      const c32 u = src[r * RS], v = src[r * RS + T];
      put(r * N, c32{u.x, u.y * imSign});
      put(r * N + T, c32{v.x, v.y * imSign});
    });
  };
  // Spectra larger than the last-level cache can hold until the contraction reads them
  // leave with the nontemporal hint (job.stream, the same for the whole launch): the
  // weight gradient of a 16 x 32 x 256 x 256 layer in 1936 windows (2 x 254 MB of spectra)
  // 310 -> 269 us; spectra that do fit (84 MB for 128 x 64 x 27 x 27 * 192 x 64 x 5 x 5)
  // lose 2-7 % with it, because the contraction then fetches them from HBM.
  auto copyOut = [&](int r0) __attribute__((always_inline)) {
    if (job.stream)
      copyOutAs(r0, std::true_type{});
    else
      copyOutAs(r0, std::false_type{});
  };

  const int ra = (wg % job.rowGroups) * GROUPS * SLOTS;
  c32 za0[H], za1[H];
  load(ra, za0, za1);
  columnPassForward<N, PAIRS == 0>(za0, za1, plane, l);
  planeSync();  // the lanes of a plane sit in one wave
  if constexpr (GROUPS == 2) {
    const int rb = ra + SLOTS;
    const bool second = rb < Rp;  // the same for the whole workgroup
    c32 zb0[H], zb1[H];
    if (second) load(rb, zb0, zb1);
    rowPassInPlace<N, true>(plane, l);
    __syncthreads();
    copyOut(ra);
    if (second) {
      __syncthreads();  // every wave has copied the first run out of the plane buffers
      columnPassForward<N, PAIRS == 0>(zb0, zb1, plane, l);
      planeSync();
      rowPassInPlace<N, true>(plane, l);
      __syncthreads();
      copyOut(rb);
    }
  } else {
    rowPassInPlace<N, true>(plane, l);
    __syncthreads();
    copyOut(ra);
  }
}

// ---- 3. C[bin][i][j] -> planes (i, j), cropped ----
// A workgroup takes GROUPS (1 or 2) runs of SLOTS consecutive j of one i.  With two, the
// second run's spectra are requested as soon as the first run's have been parked in
// LDS, and fly under the first run's transforms and stores.
template <int N, bool ACC, int GROUPS, int PAIRS>
__global__ __launch_bounds__(kTF) void inverseBinMajor(const float2* Cs, int I, int Jp, PlaneSet out,
                                                       float scale, int splits, long splitStride,
                                                       int runGroups) {
  using C = BMCfg<N>;
  constexpr int H = C::H, T = C::T, SLOTS = C::SLOTS, RS = C::RS, PSZ = C::PSZ;
  constexpr int PER = C::BINS / T;
  static_assert(C::BINS % T == 0, "bins divide evenly over the lane groups");
  __shared__ __align__(16) c32 lds[SLOTS * PSZ];
  const int t = threadIdx.x;
  const int s = t / T, l = t % T;
  // one grid index for (i, group of runs), runs fastest: a batch on i may exceed what a
  // second grid dimension can count
  const int i = blockIdx.x / runGroups, runGroup = blockIdx.x % runGroups;
  const int sp = t % SLOTS, bq = t / SLOTS;
  const long binStride = (long)I * Jp;
  c32* plane = lds + s * PSZ;

  // gather: every load of a run is issued before its first LDS store
  auto request = [&](int j0, c32 (&in)[PER]) __attribute__((always_inline)) {
    const float2* src = Cs + (long)i * Jp + j0 + sp;
    staticFor<PER>([&](auto uu) {
      constexpr int u = decltype(uu)::value;
      in[u] = src[(bq + T * u) * binStride];
    });
    // partial products of a reduction cut into ranges: added in range order
    for (int sp2 = 1; sp2 < splits; ++sp2) {
      src += splitStride;
      staticFor<PER>([&](auto uu) {
        constexpr int u = decltype(uu)::value;
        const c32 v = src[(bq + T * u) * binStride];
        in[u].x += v.x;
        in[u].y += v.y;
      });
    }
  };
  auto park = [&](const c32 (&in)[PER]) __attribute__((always_inline)) {
    c32* dstp = lds + sp * PSZ;
    staticFor<PER>([&](auto uu) {
      constexpr int u = decltype(uu)::value;  // bin = bq + T*u: row u/2, column bq + T*(u%2)
      dstp[(u / 2) * RS + T * (u % 2) + bq] = in[u];
    });
  };
  auto transformAndStore = [&](int j0) __attribute__((always_inline)) {
    // where the result goes: asked for up front, so that a described set's descriptor
    // (device memory) arrives under the transforms instead of ahead of the stores
    const int j = j0 + s;
    const PlaneWindow win = planeWindow<PAIRS == 2>(out, i, min(j, out.K - 1));
    {  // virtual bins of row 0 back to the packed row: Q[x] = C0[x] + i CH[x],
       // Q[N-x] = conj(C0[x]) + i conj(CH[x]); lane 0 sorts the four real values into
       // Q[0] = (C0[0], CH[0]) and Q[N/2] = (C0[N/2], CH[N/2]).  The T lanes of a plane
       // sit in one wave: all of them have read before any of them writes.
      const c32 c0 = plane[l], cH = plane[T + l];
      c32 q = c32{c0.x - cH.y, c0.y + cH.x}, qm = c32{c0.x + cH.y, cH.x - c0.y};
      if (l == 0) {
        q = c32{c0.x, cH.x};
        qm = c32{c0.y, cH.y};
      }
      plane[l] = q;
      plane[l == 0 ? H : N - l] = qm;
    }
    planeSync();
    rowPassInPlace<N, false>(plane, l);
    planeSync();
    c32 z0[H], z1[H];
    // PAIRS = 0, no 8-byte stores: a lane takes columns l and l + N/2, so that each store
    // instruction writes a contiguous run per plane (configs[3]: 102.4 -> 101.5 us).
    // PAIRS = 2 (described sets): columns 2l and 2l + 1, 8-byte or 4-byte stores decided
    // per plane.
    columnPassInverse<N, PAIRS == 0>(plane, l, z0, z1);
    // (Parking the cropped planes in LDS and writing them out as 16-byte runs - one
    // contiguous stream for dense outputs, row quads for windows of a tiled image - was
    // measured and is slower, 35.9 -> 36.6 us at configs[3] and 112 -> 131 us at
    // configs[4]: the kernel waits on its own chain of phases, not on store requests.
    // The dense case again with each wave parking its own four planes - one aligned run
    // of memory, no workgroup barrier - and nontemporal 16-byte stores: 106.8-108.3 us
    // per forward pass at configs[3] against 106.7-108.2, no change.)
    if (j < out.K) {  // out.K: number of valid output planes along j
      if (win.valid) {
        if constexpr (PAIRS == 2) {
          if (windowMovesAsPairs(win.p, win.sy, win.sx, win.w, win.padL))
            storeColumnsWindow<N, ACC, false, true, false>(win.p, win.sy, win.sx, win.h, win.w,
                                                           win.padL, win.padU, l, z0, z1, scale);
          else
            storeColumnsWindow<N, ACC, false, false, false>(win.p, win.sy, win.sx, win.h, win.w,
                                                            win.padL, win.padU, l, z0, z1, scale);
        } else {
          storeColumnsWindow<N, ACC, false, PAIRS == 1, PAIRS == 0>(
              win.p, win.sy, win.sx, win.h, win.w, win.padL, win.padU, l, z0, z1, scale);
        }
      }
    }
  };

  const int ja = runGroup * GROUPS * SLOTS;
  c32 in[PER];
  request(ja, in);
  park(in);
  __syncthreads();
  if constexpr (GROUPS == 2) {
    const int jb = ja + SLOTS;
    const bool second = jb < Jp;  // the same for the whole workgroup
    if (second) request(jb, in);
    transformAndStore(ja);
    if (second) {
      __syncthreads();  // every wave has read the first run out of the plane buffers
      park(in);
      __syncthreads();
      transformAndStore(jb);
    }
  } else {
    transformAndStore(ja);
  }
}

// ---- 2. batched complex GEMM, bin-major ----
constexpr int GI = 128;

struct GemmArgs {
  const float2* A;  // [bins][Kp][Ip]
  const float2* B;  // [bins][Kp][Jp]
  float2* C;        // [bins][I][Jp]
  int bins, I, Ip, Jp, Kp;
  int IT, JT;       // tiles per bin
  int N;            // transform size: bins 0 and N/2 hold pairs of real values
  // register kernels only: the reduction is cut into `splits` ranges of slicesPerSplit
  // k-slices (blockIdx.y names the range); range s writes its partial product to
  // C + s * splitStride and the inverse kernel adds the partials in range order
  int splits, slicesPerSplit;
  long splitStride;
};

// The k-slices go from HBM straight into LDS (global_load_lds, 16 bytes per lane,
// no staging registers or LDS store instructions) through a ring of three stages:
// slice s+2 is requested before slice s is multiplied, one barrier per slice.  A
// wave instruction moves 1 KiB: one k-row of 128 complex or two k-rows of 64
// complex; LDS has exactly the HBM layout.  Requires Kp % 8 == 0 with the padding
// rows zeroed; rows / columns beyond Ip / Jp are clamped (they only feed
// accumulators that are never stored).
constexpr int GJ2 = 64, GK2 = 8;

// A wave-uniform address, pinned in scalar registers: the empty statement keeps the
// compiler from folding it into a lane's offset, so that "scalar base + 32-bit lane
// offset" reaches the memory instruction as its two operands and costs no vector
// arithmetic.
template <class T>
__device__ __forceinline__ T* scalarBase(T* p) {
  asm volatile("" : "+s"(p));
  return p;
}

// ... and a lane's 32-bit offset kept apart from it up to the instruction (otherwise its
// widening to 64 bits is hoisted and the sum becomes a vector addition per access).
// (By value: the copy costs a move per access.  Marking the long-lived register itself
// instead saves the moves and measured 1.5 us slower on the weight gradient of a
// 128 x 64 x 27 x 27 * 192 x 64 x 5 x 5 layer, the same elsewhere.)
__device__ __forceinline__ unsigned laneOffset(unsigned o) {
  asm volatile("" : "+v"(o));
  return o;
}

// plain vectors in global memory (float2's members take a generic `this`)
typedef float __attribute__((ext_vector_type(2))) PlainPair;
typedef __attribute__((address_space(1))) PlainPair GlobalPair;
typedef float __attribute__((ext_vector_type(4))) PlainQuad;
typedef __attribute__((address_space(1))) PlainQuad GlobalQuad;

__device__ __forceinline__ void loadToLds(const float2* src, float2* ldsWaveBase) {
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                   (__attribute__((address_space(3))) void*)ldsWaveBase, 16, 0, 0);
}

template <int TI>
struct GemmStage {
  float2 A[GK2][TI];
  float2 B[GK2][GJ2];
};

// TI = 128: wave w owns rows 32w.. and both 32-column halves of the 64 columns.
// TI = 64 (few rows, or too few 128-row tiles to balance the chip): wave w owns rows
// 32 (w % 2).. and columns 32 (w / 2)..
template <int TI>
__global__ __launch_bounds__(kT, TI == 128 ? 4 : 6) void binGemmDirect(GemmArgs g) {
  static_assert(TI == 128 || TI == 64, "tile rows");
  constexpr int NQ = TI == 128 ? 2 : 1;
  constexpr int LOADS = TI == 128 ? 3 : 2;  // global->LDS instructions per wave and slice
  using Stage = GemmStage<TI>;
  // three separate variables, not one array: the compiler tracks pending
  // global->LDS loads per LDS variable, so reading one stage does not wait for the
  // loads still in flight into the other three
  __shared__ __align__(16) Stage stage0, stage1, stage2;
  const int t = threadIdx.x;
  const int lane = t % 64;
  // the wave's number in a scalar register: everything below that depends only on it
  // (LDS destinations, row offsets of the loads and of the result) is scalar arithmetic
  const int w = __builtin_amdgcn_readfirstlane(t / 64);
  const int r = lane % 32, h = lane / 32;

  const int total = g.bins * g.IT * g.JT;
  const int per = (total + 7) / 8;
  const int logical = (blockIdx.x % 8) * per + blockIdx.x / 8;
  if (logical >= total) return;
  const int bin = logical / (g.IT * g.JT);
  const int rem = logical % (g.IT * g.JT);
  const int i0 = (rem / g.JT) * TI, j0 = (rem % g.JT) * GJ2;
  const int rb = TI == 128 ? w : w % 2;  // 32-row block of this wave
  const int cb = TI == 128 ? 0 : w / 2;  // first 32-column block of this wave
  // bins of real pairs: (ar br, ai bi) instead of a complex product; k1 and k3 hold them
  const bool pairs = bin == 0 || 2 * bin == g.N;
  const float cross = pairs ? 0.f : 1.f;

  // this workgroup's range of the reduction (blockIdx.y; no range is empty)
  const int sliceFirst = blockIdx.y * g.slicesPerSplit;
  const float2* Ab = g.A + ((long)bin * g.Kp + (long)sliceFirst * GK2) * g.Ip;
  const float2* Bb = g.B + ((long)bin * g.Kp + (long)sliceFirst * GK2) * g.Jp;
  // per-lane source columns, clamped into the padded arrays
  const int ia = min(i0 + 2 * (TI == 128 ? lane : lane % 32), g.Ip - 2);
  const int jb = min(j0 + 2 * (lane % 32), g.Jp - 2);

  // Three real products per complex product instead of four: with a = ar + i ai and
  // b = br + i bi,  a conj(b) = (k1 - k3) + i (k1 + k2)  for
  //   k1 = (ar + ai) br,  k2 = -ar (br + bi),  k3 = ai (br - bi).
  // The sums cost three VALU adds per operand pair; the matrix pipeline, which
  // bounds this kernel, does a quarter less work.
  // (Cleared by 48 moves per sub-tile.  Giving the first slice's products a constant
  // zero addend instead takes that slice out of the loop, and there the compiler waits
  // for every load in flight before the first LDS read: 101 -> 107 us on a
  // 128 x 64 x 27 x 27 * 192 x 64 x 5 x 5 forward pass.)
  floatx16 k1[NQ], k2[NQ], k3[NQ];
#pragma unroll
  for (int q = 0; q < NQ; ++q)
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      k1[q][v] = 0.f;
      k2[q][v] = 0.f;
      k3[q][v] = 0.f;
    }

  const int slices = min(g.slicesPerSplit, g.Kp / GK2 - sliceFirst);
  // wave w moves rows 2w, 2w+1 of A and rows 2w, 2w+1 of B of a slice: LOADS instructions.
  // An address is a scalar base (slice and wave) plus a lane's 32-bit byte offset that
  // never changes, so a step spends no vector instructions on addresses.
  const unsigned laneA = (unsigned)((TI == 128 ? 0 : h * g.Ip) + ia) * (unsigned)sizeof(float2);
  const unsigned laneB = (unsigned)(h * g.Jp + jb) * (unsigned)sizeof(float2);
  const char* const waveA = (const char*)(Ab + (long)(2 * w) * g.Ip);
  const char* const waveB = (const char*)(Bb + (long)(2 * w) * g.Jp);
  const long sliceA = (long)GK2 * g.Ip * sizeof(float2), sliceB = (long)GK2 * g.Jp * sizeof(float2);
  auto issue = [&](Stage& st, int sl) __attribute__((always_inline)) {
    loadToLds((const float2*)(scalarBase(waveA + sl * sliceA) + laneOffset(laneA)), &st.A[2 * w][0]);
    if constexpr (TI == 128)
      loadToLds((const float2*)(scalarBase(waveA + sl * sliceA + g.Ip * sizeof(float2)) + laneOffset(laneA)),
                &st.A[2 * w + 1][0]);
    loadToLds((const float2*)(scalarBase(waveB + sl * sliceB) + laneOffset(laneB)), &st.B[2 * w][0]);
  };

  // One slice: wait for it, let everybody see it, request the slice two ahead into
  // the stage that was multiplied last time round, multiply.  Every step issues
  // exactly LOADS loads (past the end it re-requests the last slice into a stage
  // nobody reads), so "all but the newest LOADS have landed" always means "slice sl
  // has landed" and the compiler can count the loads in flight at every LDS read.
  // (Three stages of 8 KB let six workgroups of the 64-row kernel share a CU, 74
  // registers per lane allowing it; a fourth stage with five workgroups measured 0.6 /
  // 0.8 / 2.5 us slower on the three passes of a 128 x 64 x 27 x 27 * 192 x 64 x 5 x 5
  // layer - while the kernel needed 89 registers and five workgroups were the most
  // either way, the fourth stage was the faster form by 2 us on the weight gradient.)
  auto step = [&](Stage& cur, Stage& refill, int sl) __attribute__((always_inline)) {
    __builtin_amdgcn_s_waitcnt(0x0F70 | LOADS);  // vmcnt(LOADS): all but the newest slice
    // ... and so have everybody else's, and slice sl-1 is consumed.  A bare barrier:
    // the fences of __syncthreads() would wait for every load in flight, and no wave
    // stores to LDS with anything but these loads.
    __builtin_amdgcn_s_barrier();
    issue(refill, min(sl + 2, slices - 1));
    float2 av[GK2 / 2], bv[GK2 / 2][NQ];
#pragma unroll
    for (int s2 = 0; s2 < GK2 / 2; ++s2) {
      av[s2] = cur.A[2 * s2 + h][32 * rb + r];
#pragma unroll
      for (int q = 0; q < NQ; ++q) bv[s2][q] = cur.B[2 * s2 + h][32 * (cb + q) + r];
    }
#pragma unroll
    for (int s2 = 0; s2 < GK2 / 2; ++s2) {
      const float2 a = av[s2];
      const float as = __builtin_fmaf(cross, a.y, a.x);
#pragma unroll
      for (int q = 0; q < NQ; ++q) {
        const float2 b = bv[s2][q];
        const float nbs = -b.x - b.y, bd = __builtin_fmaf(cross, b.x, -b.y);
        k1[q] = __builtin_amdgcn_mfma_f32_32x32x2f32(as, b.x, k1[q], 0, 0, 0);
        k2[q] = __builtin_amdgcn_mfma_f32_32x32x2f32(a.x, nbs, k2[q], 0, 0, 0);
        k3[q] = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, bd, k3[q], 0, 0, 0);
      }
    }
  };

  issue(stage0, 0);
  issue(stage1, min(1, slices - 1));
  int sl = 0;
  for (; sl + 3 <= slices; sl += 3) {
    step(stage0, stage2, sl);
    step(stage1, stage0, sl + 1);
    step(stage2, stage1, sl + 2);
  }
  if (sl < slices) {
    step(stage0, stage2, sl);
    if (sl + 1 < slices) step(stage1, stage0, sl + 1);
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): nothing may land in LDS after this wave is gone

  // The sums leave unscaled; the inverse transform's factor carries 1 / N^2.
  float2* Cb = g.C + blockIdx.y * g.splitStride + (long)bin * g.I * g.Jp;
  if (i0 + 32 * rb + 32 <= g.I && j0 + 32 * (cb + NQ) <= g.Jp) {
    // the wave's whole block lies inside C: a scalar base per accumulator row plus the
    // lane's fixed offset, no tests
    const unsigned laneC = (unsigned)(4 * h * g.Jp + r) * (unsigned)sizeof(float2);
    char* const waveC = (char*)(Cb + (long)(i0 + 32 * rb) * g.Jp + j0 + 32 * cb);
    const long rowC = (long)g.Jp * sizeof(float2);
    auto store = [&](auto realPairs) __attribute__((always_inline)) {
#pragma unroll
      for (int q = 0; q < NQ; ++q)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          // (global address space spelled out: behind the pinned base the compiler no
          // longer sees where the pointer came from and would store through flat addresses)
          typedef float __attribute__((ext_vector_type(2))) Pair;  // a plain vector: float2's assignment takes a generic `this`
          auto* dst = (__attribute__((address_space(1))) Pair*)(
              scalarBase(waveC + (8 * (v / 4) + v % 4) * rowC + q * 32 * (long)sizeof(float2)) +
              laneOffset(laneC));
          if constexpr (decltype(realPairs)::value)
            *dst = Pair{k1[q][v], -k3[q][v]};
          else
            *dst = Pair{k1[q][v] - k3[q][v], k1[q][v] + k2[q][v]};
        }
    };
    if (pairs)
      store(std::true_type{});
    else
      store(std::false_type{});
    return;
  }
#pragma unroll
  for (int q = 0; q < NQ; ++q) {
    const int j = j0 + 32 * (cb + q) + r;
    if (j >= g.Jp) continue;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int i = i0 + 32 * rb + 8 * (v / 4) + 4 * h + v % 4;
      if (i < g.I)
        Cb[(long)i * g.Jp + j] = pairs ? float2{k1[q][v], -k3[q][v]}
                                       : float2{k1[q][v] - k3[q][v], k1[q][v] + k2[q][v]};
    }
  }
}

// The same product with no LDS in the loop and no barriers there: a wave loads exactly
// the operand values its own MFMA lanes supply - lane (r, h) of v_mfma_f32_32x32x2_f32
// supplies row / column r at k = h, so one 8-byte load per lane fetches k-rows 2s and
// 2s+1 of 32 consecutive rows (two 256-byte runs per wave instruction).  Slices of 8 k
// ride a ring of three register sets, two in flight while one is multiplied; the
// scheduling barriers keep each slice's loads ahead of the products of the slice two
// before it (left alone the compiler sinks the loads below the products and then waits
// for all of them at the top of the loop).
template <class Slice, class Fetch, class Multiply>
__device__ __forceinline__ void ringOfThree(int first, int step, int n, Fetch fetch,
                                            Multiply multiply) {
  // slices first, first + step, ...: n of them
  if (n <= 0) return;
  Slice s0, s1, s2;
  fetch(s0, first);
  fetch(s1, first + step * min(1, n - 1));
  int sl = 0;
  for (; sl + 3 <= n; sl += 3) {
    fetch(s2, first + step * min(sl + 2, n - 1));
    __builtin_amdgcn_sched_barrier(0);
    multiply(s0);
    __builtin_amdgcn_sched_barrier(0);
    fetch(s0, first + step * min(sl + 3, n - 1));
    __builtin_amdgcn_sched_barrier(0);
    multiply(s1);
    __builtin_amdgcn_sched_barrier(0);
    fetch(s1, first + step * min(sl + 4, n - 1));
    __builtin_amdgcn_sched_barrier(0);
    multiply(s2);
    __builtin_amdgcn_sched_barrier(0);
  }
  if (sl < n) {
    multiply(s0);
    if (sl + 1 < n) multiply(s1);
  }
}

// The same with two register sets: one slice in flight while one is multiplied.
template <class Slice, class Fetch, class Multiply>
__device__ __forceinline__ void ringOfTwo(int first, int step, int n, Fetch fetch, Multiply multiply) {
  if (n <= 0) return;
  Slice s0, s1;
  fetch(s0, first);
  int sl = 0;
  for (; sl + 2 <= n; sl += 2) {
    fetch(s1, first + step * (sl + 1));
    __builtin_amdgcn_sched_barrier(0);
    multiply(s0);
    __builtin_amdgcn_sched_barrier(0);
    fetch(s0, first + step * min(sl + 2, n - 1));
    __builtin_amdgcn_sched_barrier(0);
    multiply(s1);
    __builtin_amdgcn_sched_barrier(0);
  }
  if (sl < n) multiply(s0);
}

// Both sides short (up to 32 rows and 32 columns per bin, any K - the weight gradient
// of a layer with few planes reduces over every image and window): one workgroup per
// bin and range of the reduction; its four waves take every fourth k-slice each and
// wave 0 adds the four 32 x 32 partial tiles in wave order (through LDS) before it
// stores, so the result does not depend on timing.
struct GemmSlice {
  float2 a[GK2 / 2], b[GK2 / 2];
};

__global__ __launch_bounds__(kT, 4) void binGemmRegsSplitK(GemmArgs g) {
  __shared__ float red[3][48][64];
  const int t = threadIdx.x;
  // (the wave's number in a scalar register: its slices and their addresses are scalar)
  const int lane = t % 64, w = __builtin_amdgcn_readfirstlane(t / 64);
  const int r = lane % 32, h = lane / 32;
  const int per = (g.bins + 7) / 8;
  const int bin = (blockIdx.x % 8) * per + blockIdx.x / 8;
  if (bin >= g.bins) return;
  const bool pairs = bin == 0 || 2 * bin == g.N;  // bins of real pairs: (ar br, ai bi)
  const float cross = pairs ? 0.f : 1.f;

  // operand columns beyond the padded arrays are clamped (they feed accumulators that
  // are never stored).  An address is a scalar base (bin, k-rows) plus the lane's fixed
  // 32-bit offset: no vector arithmetic per load.
  const unsigned laneA = (unsigned)(h * g.Ip + min(r, g.Ip - 1)) * (unsigned)sizeof(float2);
  const unsigned laneB = (unsigned)(h * g.Jp + min(r, g.Jp - 1)) * (unsigned)sizeof(float2);
  const char* const binA = (const char*)(g.A + (long)bin * g.Kp * g.Ip);
  const char* const binB = (const char*)(g.B + (long)bin * g.Kp * g.Jp);
  const long sa = 2L * g.Ip * sizeof(float2), sb = 2L * g.Jp * sizeof(float2);  // two k-rows

  floatx16 k1, k2, k3;
#pragma unroll
  for (int v = 0; v < 16; ++v) k1[v] = k2[v] = k3[v] = 0.f;

  auto fetch = [&](GemmSlice& s, int sl) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < GK2 / 2; ++u) {
      const long k2rows = (long)sl * (GK2 / 2) + u;
      const PlainPair va = *(const GlobalPair*)(scalarBase(binA + k2rows * sa) + laneOffset(laneA));
      const PlainPair vb = *(const GlobalPair*)(scalarBase(binB + k2rows * sb) + laneOffset(laneB));
      s.a[u] = float2{va.x, va.y};
      s.b[u] = float2{vb.x, vb.y};
    }
  };
  // a conj(b) = (k1 - k3) + i (k1 + k2) with k1 = (ar + ai) br, k2 = -ar (br + bi),
  // k3 = ai (br - bi)
  auto multiply = [&](const GemmSlice& s) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < GK2 / 2; ++u) {
      const float2 a = s.a[u], b = s.b[u];
      k1 = __builtin_amdgcn_mfma_f32_32x32x2f32(__builtin_fmaf(cross, a.y, a.x), b.x, k1, 0, 0, 0);
      k2 = __builtin_amdgcn_mfma_f32_32x32x2f32(a.x, -b.x - b.y, k2, 0, 0, 0);
      k3 = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, __builtin_fmaf(cross, b.x, -b.y), k3, 0, 0, 0);
    }
  };
  const int slices = g.Kp / GK2;
  const int rangeFirst = blockIdx.y * g.slicesPerSplit;
  const int rangeEnd = min(rangeFirst + g.slicesPerSplit, slices);
  // wave w takes slices w, w + 4, ... of the range: the workgroup reads one front
  const int first = rangeFirst + w;
  ringOfThree<GemmSlice>(first, 4, first < rangeEnd ? (rangeEnd - first + 3) / 4 : 0, fetch,
                         multiply);

  if (w > 0) {
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      red[w - 1][v][lane] = k1[v];
      red[w - 1][16 + v][lane] = k2[v];
      red[w - 1][32 + v][lane] = k3[v];
    }
  }
  __syncthreads();
  if (w > 0) return;
#pragma unroll 1
  for (int u = 0; u < 3; ++u)
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      k1[v] += red[u][v][lane];
      k2[v] += red[u][16 + v][lane];
      k3[v] += red[u][32 + v][lane];
    }
  float2* Cb = g.C + blockIdx.y * g.splitStride + (long)bin * g.I * g.Jp;
  if (r < g.Jp) {
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int i = 8 * (v / 4) + 4 * h + v % 4;
      if (i < g.I)
        Cb[(long)i * g.Jp + r] =
            pairs ? float2{k1[v], -k3[v]} : float2{k1[v] - k3[v], k1[v] + k2[v]};
    }
  }
}

// The register kernel for products with a short side (up to 32 rows of C per bin; the
// host puts the short side on i): a wave owns 32 rows x 64 columns.  Lane (r, h) loads
// 16 bytes of B per k-pair - columns j0 + 2r and j0 + 2r + 1 at k = 2s + h - which feed two
// MFMA sub-tiles with interleaved columns, and stores the two results of a row side by
// side as 16 bytes: half the memory instructions of two 32 x 32 sub-tiles, 512-byte runs,
// and A (small, shared by every wave of the bin) is read once per 64 columns.  The four
// waves of a workgroup take consecutive column blocks.
struct GemmSliceWide {
  float2 a[GK2 / 2];
  float4 b[GK2 / 2];
};

__global__ __launch_bounds__(kT, 3) void binGemmRegsWide(GemmArgs g) {
  const int t = threadIdx.x;
  const int lane = t % 64, w = __builtin_amdgcn_readfirstlane(t / 64);
  const int r = lane % 32, h = lane / 32;
  // g.IT: 32-row blocks, g.JT: workgroups (4 x 64 columns) along j
  const int total = g.bins * g.IT * g.JT;
  const int per = (total + 7) / 8;
  const int logical = (blockIdx.x % 8) * per + blockIdx.x / 8;
  if (logical >= total) return;
  const int bin = logical / (g.IT * g.JT);
  const int rem = logical % (g.IT * g.JT);
  const int i0 = (rem / g.JT) * 32, j0 = ((rem % g.JT) * 4 + w) * 64;
  if (j0 >= g.Jp) return;
  const bool pairs = bin == 0 || 2 * bin == g.N;  // bins of real pairs: (ar br, ai bi)
  const float cross = pairs ? 0.f : 1.f;

  // operand columns beyond the padded arrays are clamped (they feed accumulators that
  // are never stored); Jp is even and rows of B and C start on 16-byte boundaries
  // (an address: a scalar base - bin, k-rows, column block - plus the lane's fixed offset)
  const unsigned laneA = (unsigned)(h * g.Ip + min(i0 + r, g.Ip - 1)) * (unsigned)sizeof(float2);
  const unsigned laneB = (unsigned)(h * g.Jp + min(2 * r, g.Jp - 2 - j0)) * (unsigned)sizeof(float2);
  const char* const binA = (const char*)(g.A + (long)bin * g.Kp * g.Ip);
  const char* const binB = (const char*)(g.B + (long)bin * g.Kp * g.Jp + j0);
  const long sa = 2L * g.Ip * sizeof(float2), sb = 2L * g.Jp * sizeof(float2);  // two k-rows

  floatx16 k1[2], k2[2], k3[2];
#pragma unroll
  for (int q = 0; q < 2; ++q)
#pragma unroll
    for (int v = 0; v < 16; ++v) k1[q][v] = k2[q][v] = k3[q][v] = 0.f;

  auto fetch = [&](GemmSliceWide& s, int sl) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < GK2 / 2; ++u) {
      const long k2rows = (long)sl * (GK2 / 2) + u;
      const PlainPair va = *(const GlobalPair*)(scalarBase(binA + k2rows * sa) + laneOffset(laneA));
      const PlainQuad vb = *(const GlobalQuad*)(scalarBase(binB + k2rows * sb) + laneOffset(laneB));
      s.a[u] = float2{va.x, va.y};
      s.b[u] = float4{vb.x, vb.y, vb.z, vb.w};
    }
  };
  // a conj(b) = (k1 - k3) + i (k1 + k2) with k1 = (ar + ai) br, k2 = -ar (br + bi),
  // k3 = ai (br - bi)
  auto multiply = [&](const GemmSliceWide& s) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < GK2 / 2; ++u) {
      const float2 a = s.a[u];
      const float as = __builtin_fmaf(cross, a.y, a.x);
      const float4 b = s.b[u];
      k1[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(as, b.x, k1[0], 0, 0, 0);
      k2[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a.x, -b.x - b.y, k2[0], 0, 0, 0);
      k3[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, __builtin_fmaf(cross, b.x, -b.y), k3[0], 0, 0, 0);
      k1[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(as, b.z, k1[1], 0, 0, 0);
      k2[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a.x, -b.z - b.w, k2[1], 0, 0, 0);
      k3[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, __builtin_fmaf(cross, b.z, -b.w), k3[1], 0, 0, 0);
    }
  };
  const int first = blockIdx.y * g.slicesPerSplit;
  // two register sets instead of three: 153 registers, three waves per SIMD instead of two
  // (configs[4]: 294.6 -> 290.1 us per forward pass)
  ringOfTwo<GemmSliceWide>(first, 1, min(first + g.slicesPerSplit, g.Kp / GK2) - first, fetch,
                           multiply);

  float2* Cb = g.C + blockIdx.y * g.splitStride + (long)bin * g.I * g.Jp;
  const int j = j0 + 2 * r;
  if (j < g.Jp) {
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int i = i0 + 8 * (v / 4) + 4 * h + v % 4;
      if (i < g.I) {
        float4 o;
        if (pairs)
          o = float4{k1[0][v], -k3[0][v], k1[1][v], -k3[1][v]};
        else
          o = float4{k1[0][v] - k3[0][v], k1[0][v] + k2[0][v], k1[1][v] - k3[1][v],
                     k1[1][v] + k2[1][v]};
        *reinterpret_cast<float4*>(Cb + (long)i * g.Jp + j) = o;
      }
    }
  }
}

inline int roundUp(int a, int b) { return (a + b - 1) / b * b; }

// Which operand takes the 128-wide side of the GEMM tile (and with it the role of i, the
// slow index of C[bin][i][j]).  Results cut into windows of a larger image (outTiled)
// always put the window index on j: the inverse kernel transforms 16 consecutive j per
// workgroup, and 16 neighbouring windows of one output plane store whole stretches of
// image rows where 16 output planes of one window store 24-float pieces 248 floats apart
// (configs[4]: 337 -> 308 us per forward pass).  Otherwise: the assignment with fewer
// padded tile elements.
inline bool swapRoles(int I, int J, bool outTiled) {
  if (outTiled) return true;
  if (I <= 32 || J <= 32) return J < I;  // the register kernel takes the short side on i
  return (long)roundUp(J, GI) * roundUp(I, GJ2) < (long)roundUp(I, GI) * roundUp(J, GJ2);
}

// Which contraction kernel runs a product, on which tiles, and into how many ranges the
// reduction is cut (range s writes its partial product to C + s * splitStride and the
// inverse kernel adds the partials in range order, so the result does not depend on
// timing).  A short side (up to 32, which the roles put on i) takes the register kernels:
// the LDS kernels' tiles would be half empty.  64-row tiles when they waste fewer rows,
// or when 128-row tiles would leave the chip with fewer than eight workgroups per CU to
// balance (measured equal or faster there: 84 -> 62 us for 64 x 192 x 128 per bin,
// 77 -> 69 us for 128 x 64 x 192).  Ranges: when the tiles alone leave most of the chip
// idle and the reduction is long - 8- and 16-point transforms have 32 and 128 bins, and a
// weight gradient reduces over every image and window - up to 16 of them, enough for
// about two waves per SIMD in the register kernels and one round of workgroups in the LDS
// kernels, each keeping at least `minSlices` k-slices (weight gradient of configs[3] on
// 8-point windows: 423 -> 238 us; 64 x 64 x 512 per bin on 16-point windows: 73 -> 63 us;
// ranges of 8 slices cost 6 % where 16 slices are all there are).  32-point transforms on short sides
// have 512 bins and never split (measured on the weight gradient of configs[4], 32 x 32
// per bin over 1936 windows, 2048 waves: two ranges 337 -> 345 us, four 362: that
// contraction is not short of waves).
struct GemmPlan {
  enum Kind { RegsSplitK, RegsWide, Direct64, Direct128 } kind;
  int IT, JT;
  int splits, slicesPerSplit;
};

inline GemmPlan planGemm(int bins, int I, int Jp, int Kp) {
  GemmPlan p;
  long waves, target;
  int minSlices;
  if (I <= 32 && Jp <= 32) {
    p.kind = GemmPlan::RegsSplitK;
    p.IT = p.JT = 1;
    waves = 4L * bins;
    target = 2048;
    minSlices = 16;
  } else if (I <= 32) {
    p.kind = GemmPlan::RegsWide;
    p.IT = 1;
    p.JT = ceilDiv(Jp, 256);
    waves = (long)bins * ceilDiv(Jp, 64);
    target = 2048;
    minSlices = 4;
  } else {
    p.JT = ceilDiv(Jp, GJ2);
    const bool small =
        roundUp(I, 64) < roundUp(I, GI) || (long)bins * ceilDiv(I, GI) * p.JT < 8 * 256;
    p.kind = small ? GemmPlan::Direct64 : GemmPlan::Direct128;
    p.IT = ceilDiv(I, small ? 64 : GI);
    waves = 4L * bins * p.IT * p.JT;
    target = 4096;
    minSlices = 16;
  }
  const int slices = Kp / GK2;
  const int want = (int)std::min<long>(16, ceilDiv(target, waves));
  const int most = std::max(1, slices / minSlices);
  p.slicesPerSplit = ceilDiv(slices, std::min(want, most));
  p.splits = ceilDiv(slices, p.slicesPerSplit);  // no range is empty
  return p;
}

template <int N>
size_t workspaceFloat2(int I, int J, int K, bool outTiled) {
  if (swapRoles(I, J, outTiled)) std::swap(I, J);
  const int SL = BMCfg<N>::SLOTS, bins = BMCfg<N>::BINS;
  const int Ip = roundUp(I, SL), Jp = roundUp(J, SL), Kp = roundUp(K, 8);
  return (size_t)bins * ((size_t)Kp * Ip + (size_t)Kp * Jp +
                         (size_t)planGemm(bins, I, Jp, Kp).splits * I * Jp);
}

// P[i][j] = scale * sum_k X[i][k] * op(Y[j][k]) for planes x(i,k), y(j,k) -> planes out(i,j);
// each PlaneSet names its first index "row" and its second "k".
template <int N>
int runPipeline(PlaneSet x, PlaneSet y, PlaneSet out, bool conjY, float scale, bool accumulate,
                float2* ws, hipStream_t s) {
  using C = BMCfg<N>;
  const int SL = C::SLOTS, bins = C::BINS;
  float xSign = 1.0f, ySign = conjY ? 1.0f : -1.0f;
  if (swapRoles(x.R, y.R, out.tiled != 0 || out.described != 0)) {
    // G[j][i] = sum_k op(Y[j]) * conj(conj X[i])
    std::swap(x, y);
    xSign = conjY ? -1.0f : 1.0f;
    ySign = -1.0f;
    std::swap(out.sRow, out.sK);
    if (out.tiled) out.tiled = 3 - out.tiled;
    if (out.described) out.described = 3 - out.described;
  }
  const int I = x.R, J = y.R, K = x.K;
  out.R = I;
  out.K = J;
  const int Ip = roundUp(I, SL), Jp = roundUp(J, SL), Kp = roundUp(K, 8);
  // every launch below counts its workgroups in one 31-bit grid index: refuse, before
  // anything runs, a layer whose transforms or contraction tiles outnumber that
  const long gridMax = 0x7fffffffL;
  if ((long)(Ip / SL + Jp / SL) * Kp > gridMax || (long)(Jp / SL) * I > gridMax ||
      (long)bins * ceilDiv(I, 32) * ceilDiv(Jp, 32) > gridMax)
    return FBFFT_UNSUPPORTED_SIZE;
  float2* SA = ws;
  float2* SB = SA + (size_t)bins * Kp * Ip;
  float2* SC = SB + (size_t)bins * Kp * Jp;

  // 1: every window of a set starts on an 8-byte boundary with an even width and pad;
  // 2: the windows are described on the device, each plane decides for itself; 0: 4 bytes
  auto movesAsPairs = [](const PlaneSet& p) {
    if (p.described) return 2;
    return windowMovesAsPairs(p.base, p.sy, p.sx, p.w, p.padL0) && p.sRow % 2 == 0 &&
                   p.sK % 2 == 0 && (!p.tiled || ((p.stepX | p.orgX | p.winW) & 1) == 0)
               ? 1
               : 0;
  };
  // Two runs per workgroup pay once the halved launch still fills every CU several
  // times over (measured: 114.5 -> 109.8 us on 3936 workgroups, 29.9 -> 33.7 us on a
  // launch a quarter of that).
  const bool two = (long)(ceilDiv(Ip / SL, 2) + ceilDiv(Jp / SL, 2)) * Kp >= 3L * 2 * computeUnits();
  // both operands' spectra against half of the 256 MiB last-level cache
  const int stream = (size_t)bins * Kp * ((size_t)Ip + Jp) * sizeof(float2) > (128u << 20);
  const ForwardJob ja{x, SA, Ip, Kp, xSign, two ? ceilDiv(Ip / SL, 2) : Ip / SL, stream},
      jb{y, SB, Jp, Kp, ySign, two ? ceilDiv(Jp / SL, 2) : Jp / SL, stream};
  const dim3 fgrid((unsigned)(ja.rowGroups + jb.rowGroups) * Kp);
  const int pa = movesAsPairs(x), pb = movesAsPairs(y);
  auto launchForward = [&](auto groups) {
    constexpr int G = decltype(groups)::value;
    auto withB = [&](auto modeA) {
      constexpr int A = decltype(modeA)::value;
      if (pb == 2)
        forwardBinMajor<N, A, 2, G><<<fgrid, dim3(kTF), 0, s>>>(ja, jb);
      else if (pb == 1)
        forwardBinMajor<N, A, 1, G><<<fgrid, dim3(kTF), 0, s>>>(ja, jb);
      else
        forwardBinMajor<N, A, 0, G><<<fgrid, dim3(kTF), 0, s>>>(ja, jb);
    };
    if (pa == 2)
      withB(std::integral_constant<int, 2>{});
    else if (pa == 1)
      withB(std::integral_constant<int, 1>{});
    else
      withB(std::integral_constant<int, 0>{});
  };
  if (two)
    launchForward(std::integral_constant<int, 2>{});
  else
    launchForward(std::integral_constant<int, 1>{});
  GemmArgs g;
  g.A = SA;
  g.B = SB;
  g.C = SC;
  g.bins = bins;
  g.N = N;
  g.I = I;
  g.Ip = Ip;
  g.Jp = Jp;
  g.Kp = Kp;
  const GemmPlan plan = planGemm(bins, I, Jp, Kp);
  g.IT = plan.IT;
  g.JT = plan.JT;
  g.splits = plan.splits;
  g.slicesPerSplit = plan.slicesPerSplit;
  g.splitStride = (long)bins * I * Jp;
  const dim3 ggrid(roundUp(bins * g.IT * g.JT, 8), g.splits);
  switch (plan.kind) {
    case GemmPlan::RegsSplitK: binGemmRegsSplitK<<<ggrid, dim3(kT), 0, s>>>(g); break;
    case GemmPlan::RegsWide: binGemmRegsWide<<<ggrid, dim3(kT), 0, s>>>(g); break;
    case GemmPlan::Direct64: binGemmDirect<64><<<ggrid, dim3(kT), 0, s>>>(g); break;
    case GemmPlan::Direct128: binGemmDirect<GI><<<ggrid, dim3(kT), 0, s>>>(g); break;
  }
  // Two runs per workgroup pay when the paired launch still fills the chip for three
  // rounds or more (two workgroups are resident per CU): 112 -> 108 us at configs[4],
  // 1936 paired workgroups; at configs[3] pairing would leave 768 workgroups, one and a
  // half rounds, and costs 35.5 -> 37.1 us.
  const bool pairedRuns = Jp / SL >= 2 && (long)ceilDiv(Jp / SL, 2) * I >= 3L * 2 * computeUnits();
  const int runGroups = pairedRuns ? ceilDiv(Jp / SL, 2) : Jp / SL;
  const dim3 igrid((unsigned)((long)runGroups * I));
  // windows whose rows start on 8-byte boundaries with an even width: a lane stores its
  // two columns of a row as one 8-byte word
  const int po = movesAsPairs(out);
  // the unnormalised transforms' 1 / N^2 (a power of two: exact) rides on the caller's factor
  const float invNorm = 1.0f / (float)(N * N);
  auto launchInverse = [&](auto acc, auto groups, auto pairs) {
    inverseBinMajor<N, decltype(acc)::value, decltype(groups)::value, decltype(pairs)::value>
        <<<igrid, dim3(kTF), 0, s>>>(SC, I, Jp, out, scale * invNorm, g.splits, g.splitStride,
                                     runGroups);
  };
  auto withPairs = [&](auto acc, auto groups) {
    if (po == 2)
      launchInverse(acc, groups, std::integral_constant<int, 2>{});
    else if (po == 1)
      launchInverse(acc, groups, std::integral_constant<int, 1>{});
    else
      launchInverse(acc, groups, std::integral_constant<int, 0>{});
  };
  auto withGroups = [&](auto acc) {
    if (pairedRuns)
      withPairs(acc, std::integral_constant<int, 2>{});
    else
      withPairs(acc, std::integral_constant<int, 1>{});
  };
  if (accumulate)
    withGroups(std::true_type{});
  else
    withGroups(std::false_type{});
  return launchStatus();
}

PlaneSet planes(float* base, const int* stride, const int* size, int rowDim, int kDim) {
  PlaneSet p{};
  p.base = base;
  p.sRow = stride[rowDim];
  p.sK = stride[kDim];
  p.sy = stride[2];
  p.sx = stride[3];
  p.h = size[2];
  p.w = size[3];
  p.R = size[rowDim];
  p.K = size[kDim];
  return p;
}

// Cuts the images of p into tilesY x tilesX windows; the index of dimension 0 (the
// image) - p's row or k - becomes the composite (image, tileY, tileX).
void tile(PlaneSet& p, bool imageIsRow, int tilesY, int tilesX, int stepY, int stepX, int orgY,
          int orgX, int winH, int winW) {
  p.tiled = imageIsRow ? 1 : 2;
  p.tilesY = tilesY;
  p.tilesX = tilesX;
  p.stepY = stepY;
  p.stepX = stepX;
  p.orgY = orgY;
  p.orgX = orgX;
  p.winH = winH;
  p.winW = winW;
  (imageIsRow ? p.R : p.K) *= tilesY * tilesX;
}

template <int N>
int runPass(int pass, const PlaneSet& x, const PlaneSet& y, const PlaneSet& out, float scale,
            bool accumulate, float2* ws, hipStream_t s) {
  return runPipeline<N>(x, y, out, /*conjY=*/pass != 1, scale, accumulate, ws, s);
}

}  // namespace

// Tiles per image of a pass: 1 when the image fits the transform.  The forward pass
// and the weight gradient walk the OUTPUT in disjoint (N-kH+1) x (N-kW+1) windows,
// the input gradient walks the INPUT (the tensor it writes) in such windows.
static void tileGrid(int pass, int N, int H, int W, int kH, int kW, int* tilesY, int* tilesX) {
  *tilesY = *tilesX = 1;
  if (H <= N && W <= N) return;
  const int stepY = N - kH + 1, stepX = N - kW + 1;
  const int spanY = pass == 1 ? H : H - kH + 1, spanX = pass == 1 ? W : W - kW + 1;
  *tilesY = ceilDiv(spanY, stepY);
  *tilesX = ceilDiv(spanX, stepX);
}

// (I, J, K) of a pass for batch B (times the tiles per image) and Cin / Cout planes
static void passDims(int pass, int B, int Cin, int Cout, int* I, int* J, int* K) {
  if (pass == 0) { *I = B; *J = Cout; *K = Cin; }
  else if (pass == 1) { *I = B; *J = Cin; *K = Cout; }
  else { *I = Cin; *J = Cout; *K = B; }
}

size_t convWorkspaceBytes(int pass, int N, int B, int Cin, int Cout, int H, int W, int kH,
                          int kW) {
  if (N > 32) return convSplitWorkspaceBytes(pass, N, B, Cin, Cout);
  int ty, tx;
  tileGrid(pass, N, H, W, kH, kW, &ty, &tx);
  if ((long)B * ty * tx > (1L << 30)) return 0;
  int I, J, K;
  passDims(pass, B * ty * tx, Cin, Cout, &I, &J, &K);
  const bool outTiled = pass != 2 && ty * tx > 1;  // the weight gradient is never tiled
  size_t n = N == 8 ? workspaceFloat2<8>(I, J, K, outTiled)
                    : N == 16 ? workspaceFloat2<16>(I, J, K, outTiled)
                              : workspaceFloat2<32>(I, J, K, outTiled);
  return n * sizeof(float2);
}

// pass 0: x = input [B][Cin][H][W], y = weight [Cout][Cin][kH][kW], out = output [B][Cout][oH][oW]
// pass 1: x = gradOutput [B][Cout][oH][oW], y = weight, out = gradInput [B][Cin][H][W]
// pass 2: x = input, y = gradOutput, out = gradWeight [Cout][Cin][kH][kW]
// strides in floats.  Images larger than the transform (N <= 32 only) are cut into
// overlapping windows that ride through the same three kernels as extra rows
// (passes 0 and 1) or extra reduction steps (pass 2).
int launchConvPass(int pass, int N, float* x, const int* xStride, const int* xSize, float* y,
                   const int* yStride, const int* ySize, float* out, const int* outStride,
                   const int* outSize, float scale, bool accumulate, void* workspace,
                   hipStream_t s) {
  if (N > 32)
    return launchConvSplit(pass, N, x, xStride, xSize, y, yStride, ySize, out, outStride, outSize,
                           scale, accumulate, workspace, s);
  PlaneSet px, py, po;
  if (pass == 0) {
    px = planes(x, xStride, xSize, 0, 1);
    py = planes(y, yStride, ySize, 0, 1);
    po = planes(out, outStride, outSize, 0, 1);
  } else if (pass == 1) {
    px = planes(x, xStride, xSize, 0, 1);
    py = planes(y, yStride, ySize, 1, 0);
    po = planes(out, outStride, outSize, 0, 1);
  } else {
    px = planes(x, xStride, xSize, 1, 0);
    py = planes(y, yStride, ySize, 1, 0);
    po = planes(out, outStride, outSize, 1, 0);
  }
  const int* in = pass == 1 ? outSize : xSize;    // the layer's input / gradInput extents
  const int* wt = pass == 2 ? outSize : ySize;    // the filter extents
  const int H = in[2], W = in[3], kH = wt[2], kW = wt[3];
  int ty, tx;
  tileGrid(pass, N, H, W, kH, kW, &ty, &tx);
  if (ty * tx > 1) {
    const int stepY = N - kH + 1, stepX = N - kW + 1;
    if (pass == 0) {
      tile(px, true, ty, tx, stepY, stepX, 0, 0, N, N);
      tile(po, true, ty, tx, stepY, stepX, 0, 0, stepY, stepX);
    } else if (pass == 1) {
      // gradInput rows y0 .. y0+step-1 are a full convolution over gradOutput rows
      // y0-(kH-1) .. y0+step-1; the result for row y0 then sits in plane row kH-1,
      // clear of the circular wrap-around
      tile(px, true, ty, tx, stepY, stepX, -(kH - 1), -(kW - 1), N, N);
      tile(po, true, ty, tx, stepY, stepX, 0, 0, stepY, stepX);
      po.padU0 = kH - 1;
      po.padL0 = kW - 1;
    } else {
      tile(px, false, ty, tx, stepY, stepX, 0, 0, N, N);
      tile(py, false, ty, tx, stepY, stepX, 0, 0, stepY, stepX);
    }
  }
  float2* ws = static_cast<float2*>(workspace);
  switch (N) {
    case 8: return runPass<8>(pass, px, py, po, scale, accumulate, ws, s);
    case 16: return runPass<16>(pass, px, py, po, scale, accumulate, ws, s);
    case 32: return runPass<32>(pass, px, py, po, scale, accumulate, ws, s);
  }
  return FBFFT_UNSUPPORTED_SIZE;
}

// FFTIteratedConvolution's operands - device arrays of tile descriptors - through the
// same three kernels: tile t of ins / outs is a [batch][planes][h][w] view with its own
// strides and pads, the (image, tile) pairs ride as rows (passes 0 and 1) or as
// reduction steps (pass 2).  Roles as in iterated_conv.hip's table: pass 0
// outs[t](n, f) = sum_c ins[t](n, c) * conj(weight(f, c)), pass 1 ins[t](n, c) =
// sum_f outs[t](n, f) * weight(f, c), pass 2 weight(f, c) = scale * sum_(t, n)
// ins[t](n, c) * conj(outs[t](n, f)); results land at (padU, padL) of the destination's
// plane.  The descriptors are only read on the device.
size_t describedWorkspaceBytes(int pass, int N, long rows, int Cin, int Cout) {
  if (rows <= 0 || rows > (1L << 30)) return 0;
  int I, J, K;
  passDims(pass, (int)rows, Cin, Cout, &I, &J, &K);
  const bool outTiled = pass != 2;
  const size_t n = N == 8 ? workspaceFloat2<8>(I, J, K, outTiled)
                          : N == 16 ? workspaceFloat2<16>(I, J, K, outTiled)
                                    : workspaceFloat2<32>(I, J, K, outTiled);
  return n * sizeof(float2);
}

int launchDescribedConv(int pass, int N, const fbfft_tile* ins, const fbfft_tile* outs, float* weight,
                        const int* wStride, const int* wSize, float scale, int batch, int numTiles,
                        void* workspace, hipStream_t s) {
  const int Cout = wSize[0], Cin = wSize[1];
  auto described = [&](const fbfft_tile* tiles, bool compositeIsRow, int planes) {
    PlaneSet p{};
    p.tiles = tiles;
    p.described = compositeIsRow ? 1 : 2;
    p.numTiles = numTiles;
    (compositeIsRow ? p.R : p.K) = numTiles * batch;
    (compositeIsRow ? p.K : p.R) = planes;
    return p;
  };
  float* w = weight;
  PlaneSet px, py, po;
  if (pass == 0) {
    px = described(ins, true, Cin);
    py = planes(w, wStride, wSize, 0, 1);
    po = described(outs, true, Cout);
  } else if (pass == 1) {
    px = described(outs, true, Cout);
    py = planes(w, wStride, wSize, 1, 0);
    po = described(ins, true, Cin);
  } else {
    px = described(ins, false, Cin);
    py = described(outs, false, Cout);
    po = planes(w, wStride, wSize, 1, 0);
  }
  float2* ws = static_cast<float2*>(workspace);
  const float sc = pass == 2 ? scale : 1.0f;
  switch (N) {
    case 8: return runPass<8>(pass, px, py, po, sc, false, ws, s);
    case 16: return runPass<16>(pass, px, py, po, sc, false, ws, s);
    case 32: return runPass<32>(pass, px, py, po, sc, false, ws, s);
  }
  return FBFFT_UNSUPPORTED_SIZE;
}

}  // namespace fbfft_amd
