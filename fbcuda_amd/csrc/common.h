// Host/device helpers shared by the kernels and the C ABI.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/fbfft_amd.h"

namespace fbfft_amd {

// real [B][h][w]; strides in floats
struct RealView {
  float* data;
  int sb, sy, sx;
  int B, h, w;
};

// complex-as-float [B][rows][cols][2]; strides in floats, (re, im) adjacent
struct CplxView {
  float* data;
  int sb, sr, sc;
  int B, rows, cols;
};

// the unsigned-compare bounds test of MemoryAccess.cuh:19-25
__host__ __device__ __forceinline__ bool inWindow(int y, int x, int padU, int padL, int h, int w) {
  return (unsigned)(y - padU) < (unsigned)h && (unsigned)(x - padL) < (unsigned)w;
}

__host__ __device__ inline int ceilDiv(int a, int b) { return (a + b - 1) / b; }

// Stores of results that the launch itself never reads back carry the nontemporal
// hint: the lines are not kept in L2 or in the 256 MiB last-level cache on their way to
// HBM, so they do not push the operands still to be read out of it.  Measured on
// batches larger than that cache: 32 x 32 R2C of 65536 planes 100.4 -> 85.9 us (5.5 ->
// 6.4 TB/s), 16 x 16 98.6 -> 87.9 us, 8 x 8 105.0 -> 86.7 us; the same hint on the loads
// costs 5 %.  Operands that stay in the cache from one launch to the next (the same
// 132 MB over and over) lose 2-3 %.
typedef float vfloat2 __attribute__((ext_vector_type(2)));
typedef float vfloat4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void streamStore(float4* p, float4 v) {
  __builtin_nontemporal_store(vfloat4{v.x, v.y, v.z, v.w}, reinterpret_cast<vfloat4*>(p));
}
__device__ __forceinline__ void streamStore(float2* p, float2 v) {
  __builtin_nontemporal_store(vfloat2{v.x, v.y}, reinterpret_cast<vfloat2*>(p));
}
__device__ __forceinline__ void streamStore(float* p, float v) {
  __builtin_nontemporal_store(v, p);
}

inline bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

// status of the launches just made; the error is consumed, so that one failed
// launch does not make every later call of the process report failure
inline int launchStatus() {
  return hipGetLastError() == hipSuccess ? FBFFT_SUCCESS : FBFFT_HIP_ERROR;
}

// compute units of the current device (256 on MI355X); queried once
inline int computeUnits() {
  static const int n = [] {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        cus <= 0)
      cus = 256;
    return cus;
  }();
  return n;
}

// kernel launchers implemented in the .hip files (return an fbfft_error)
int launchFft2dSmallForward(int N, const RealView& real, const CplxView& cplx, int padL, int padU,
                            hipStream_t s, bool packed = false);
int launchFft2dSmallInverse(int N, const CplxView& cplx, const RealView& real, int padL, int padU,
                            hipStream_t s, bool packed = false);

int launchFft2dTinyForward(int N, const RealView& real, const CplxView& cplx, int padL, int padU,
                           hipStream_t s);
int launchFft2dTinyInverse(int N, const CplxView& cplx, const RealView& real, int padL, int padU,
                           hipStream_t s);

int launchFft2dLargeForward(int N, const RealView& real, const CplxView& cplx, int padL, int padU,
                            hipStream_t s);
int launchFft2dLargeInverse(int N, const CplxView& cplx, const RealView& real, int padL, int padU,
                            hipStream_t s);

int launchFft1d(bool forward, int N, float* real, int sb, int sx, float* cplx, int cb, int ck,
                int B, int padL, hipStream_t s);

int launchTransposeMM(const float* A, long a0, long a1, const float* B, long b0, long b1, float* C,
                      long c0, long c1, int I, int J, int K, int XY, bool conjA, bool conjB,
                      bool accumulate, float invNorm, hipStream_t s);

int launchTransposeMMPacked(const float* A, long a0, long a1, const float* B, long b0, long b1,
                            float* C, long c0, long c1, int I, int J, int K, int N, bool conjA,
                            bool conjB, bool accumulate, float invNorm, hipStream_t s);

int launchIteratedConv(int N, const fbfft_tile* ins, const fbfft_tile* outs, float* weight,
                       const int* wStride, const int* wSize, int pass, float scale, int batch,
                       size_t numTiles, bool deterministic, hipStream_t s);

// mode 0/1: forward pass 1/2, mode 2/3: inverse pass 1/2 of the two-call 64/128 forms
int launchTwoPass(int N, int mode, float* src, long s0, long s1, long s2, float* dst, long d0,
                  long d1, long d2, int B, int h, int w, int padL, int padU, hipStream_t s);

// pass 0 / 1 / 2 = forward, input gradient, weight gradient (x, y, out as in conv_pipeline.hip)
// H, W: the layer's input extents (larger than N: overlap tiling, N <= 32 only)
size_t convWorkspaceBytes(int pass, int N, int B, int Cin, int Cout, int H, int W, int kH, int kW);
size_t describedWorkspaceBytes(int pass, int N, long rows, int Cin, int Cout);
int launchDescribedConv(int pass, int N, const fbfft_tile* ins, const fbfft_tile* outs, float* weight,
                        const int* wStride, const int* wSize, float scale, int batch, int numTiles,
                        void* workspace, hipStream_t s);
int launchConvPass(int pass, int N, float* x, const int* xStride, const int* xSize, float* y,
                   const int* yStride, const int* ySize, float* out, const int* outStride,
                   const int* outSize, float scale, bool accumulate, void* workspace,
                   hipStream_t s);

// the same passes for 64- and 128-point transforms (conv_split.hip)
size_t convSplitWorkspaceBytes(int pass, int N, int B, int Cin, int Cout);
int launchConvSplit(int pass, int N, float* x, const int* xStride, const int* xSize, float* y,
                    const int* yStride, const int* ySize, float* out, const int* outStride,
                    const int* outSize, float scale, bool accumulate, void* workspace,
                    hipStream_t s);

}  // namespace fbfft_amd
