// Convolution-layer passes for 64- and 128-point transforms.
//
// Planes of that size do not fit the one-workgroup-per-plane-group forward and
// inverse kernels of the bin-major pipeline, so these sizes run the composition the
// reference's external callers run (MM-inl.cuh:188-196): fbfft2D of both operands
// into plane-major half spectra [d0][d1][N/2+1][N], transposeMM with the role's
// conjugation, fbifft2D with crop on store.  All three stages are this library's
// own kernels (fft2dLargeForward, transposeMMKernel, fft2dLargeInverse); the
// spectra live in the caller's workspace and cross HBM once each way.
#include "common.h"

namespace fbfft_amd {
namespace {

struct Planes4 {
  float* data;
  const int* stride;
  const int* size;
};

// [d0][d1] collapses into one batch index when one of them is 1 or dim 0 steps over
// exactly d1 planes
bool collapses(const Planes4& t) {
  return t.size[0] == 1 || t.size[1] == 1 ||
         (long)t.stride[0] == (long)t.size[1] * t.stride[1];
}

inline long specFloats(int N) { return (long)(N / 2 + 1) * N * 2; }

// calls f(realView, spectrum of the first plane of the view) once for the whole
// tensor, or once per index of dim 0 when the planes do not form one batch
template <class F>
int forPlaneBatches(int N, const Planes4& t, float* spec, F f) {
  const long plane = specFloats(N);
  const int d0 = t.size[0], d1 = t.size[1];
  if (collapses(t)) {
    const int sb = d1 == 1 ? t.stride[0] : t.stride[1];
    RealView r{t.data, sb, t.stride[2], t.stride[3], d0 * d1, t.size[2], t.size[3]};
    return f(r, spec);
  }
  for (int i = 0; i < d0; ++i) {
    RealView r{t.data + (long)i * t.stride[0], t.stride[1], t.stride[2], t.stride[3], d1,
               t.size[2], t.size[3]};
    const int rc = f(r, spec + (long)i * d1 * plane);
    if (rc != FBFFT_SUCCESS) return rc;
  }
  return FBFFT_SUCCESS;
}

CplxView specView(int N, float* spec, int B) {
  return CplxView{spec, (int)specFloats(N), 2 * N, 2, B, N / 2 + 1, N};
}

int forwardAll(int N, const Planes4& t, float* spec, hipStream_t s) {
  return forPlaneBatches(N, t, spec, [&](const RealView& r, float* sp) {
    return launchFft2dLargeForward(N, r, specView(N, sp, r.B), 0, 0, s);
  });
}

int inverseAll(int N, float* spec, const Planes4& t, hipStream_t s) {
  return forPlaneBatches(N, t, spec, [&](const RealView& r, float* sp) {
    return launchFft2dLargeInverse(N, specView(N, sp, r.B), r, 0, 0, s);
  });
}

// out[a][b][y][x] += tmp[a][b][y][x] (tmp contiguous)
__global__ void addPlanes(float* out, long s0, long s1, long s2, long s3, int d1, int d2, int d3,
                          const float* tmp, long n) {
  for (long q = (long)blockIdx.x * blockDim.x + threadIdx.x; q < n;
       q += (long)gridDim.x * blockDim.x) {
    long r = q;
    const int x = r % d3;
    r /= d3;
    const int y = r % d2;
    r /= d2;
    const int b = r % d1;
    const long a = r / d1;
    out[a * s0 + b * s1 + y * s2 + x * s3] += tmp[q];
  }
}

}  // namespace

size_t convSplitWorkspaceBytes(int pass, int N, int B, int Cin, int Cout) {
  const size_t planes = (size_t)B * Cin + (size_t)Cout * Cin + (size_t)B * Cout;
  size_t floats = planes * specFloats(N);
  if (pass == 2) floats += (size_t)Cout * Cin * N * N;  // staging for an accumulating store
  return floats * sizeof(float);
}

// x, y, out as in launchConvPass
int launchConvSplit(int pass, int N, float* x, const int* xStride, const int* xSize, float* y,
                    const int* yStride, const int* ySize, float* out, const int* outStride,
                    const int* outSize, float scale, bool accumulate, void* workspace,
                    hipStream_t s) {
  const Planes4 px{x, xStride, xSize}, py{y, yStride, ySize}, po{out, outStride, outSize};
  const long plane = specFloats(N);
  float* SX = static_cast<float*>(workspace);
  float* SY = SX + (long)xSize[0] * xSize[1] * plane;
  float* SO = SY + (long)ySize[0] * ySize[1] * plane;
  float* tmp = SO + (long)outSize[0] * outSize[1] * plane;

  int rc = forwardAll(N, px, SX, s);
  if (rc != FBFFT_SUCCESS) return rc;
  rc = forwardAll(N, py, SY, s);
  if (rc != FBFFT_SUCCESS) return rc;

  const int XY = (N / 2 + 1) * N;
  const float invNorm = scale / (float)(N * N);
  const long x0 = (long)xSize[1] * plane, y0 = (long)ySize[1] * plane,
             o0 = (long)outSize[1] * plane;
  if (pass == 0) {
    // output[b][co] = sum_ci input[b][ci] * conj(weight[co][ci])
    rc = launchTransposeMM(SX, x0, plane, SY, y0, plane, SO, o0, plane, xSize[0], ySize[0],
                           xSize[1], XY, false, true, false, invNorm, s);
  } else if (pass == 1) {
    // gradInput[b][ci] = sum_co gradOutput[b][co] * weight[co][ci]
    rc = launchTransposeMM(SX, x0, plane, SY, y0, plane, SO, o0, plane, xSize[0], ySize[1],
                           xSize[1], XY, false, false, false, invNorm, s);
  } else {
    // gradWeight[co][ci] = sum_b conj(gradOutput[b][co]) * input[b][ci]
    rc = launchTransposeMM(SY, y0, plane, SX, x0, plane, SO, o0, plane, ySize[1], xSize[1],
                           xSize[0], XY, true, false, false, invNorm, s);
  }
  if (rc != FBFFT_SUCCESS) return rc;

  if (!accumulate) return inverseAll(N, SO, po, s);

  const int contiguous[4] = {outSize[1] * outSize[2] * outSize[3], outSize[2] * outSize[3],
                             outSize[3], 1};
  rc = inverseAll(N, SO, Planes4{tmp, contiguous, outSize}, s);
  if (rc != FBFFT_SUCCESS) return rc;
  const long n = (long)outSize[0] * contiguous[0];
  const int blocks = (int)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096);
  addPlanes<<<dim3(blocks), dim3(256), 0, s>>>(out, outStride[0], outStride[1], outStride[2],
                                               outStride[3], outSize[1], outSize[2], outSize[3],
                                               tmp, n);
  return launchStatus();
}

}  // namespace fbfft_amd
