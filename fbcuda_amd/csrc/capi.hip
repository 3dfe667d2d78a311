// C ABI: argument validation and dispatch.  Nothing here touches device memory
// or synchronises; every kernel is enqueued on the caller's stream.
#include <string.h>

#include "common.h"

#include <algorithm>
#include "fft_regs.h"

using namespace fbfft_amd;

namespace {

bool isPow2(int n) { return n > 0 && (n & (n - 1)) == 0; }

bool okTensor(const fbfft_tensor* t, int dim) {
  if (!t || t->dim != dim) return false;
  for (int d = 0; d < dim; ++d)
    if (t->size[d] < 0) return false;
  return true;
}

bool empty(const fbfft_tensor* t) {
  for (int d = 0; d < t->dim; ++d)
    if (t->size[d] == 0) return true;
  return false;
}

RealView realView3(const fbfft_tensor* t) {
  return RealView{t->data, t->stride[0], t->stride[1], t->stride[2],
                  t->size[0], t->size[1], t->size[2]};
}

// [B][rows][cols][2]
CplxView cplxView4(const fbfft_tensor* t) {
  return CplxView{t->data, t->stride[0], t->stride[1], t->stride[2],
                  t->size[0], t->size[1], t->size[2]};
}

// complex-as-float operands must keep (re, im) adjacent, 8-byte aligned, and
// every stride even so that each element can be moved as one 8-byte word
bool okCplx(const fbfft_tensor* t) {
  const int d = t->dim;
  if (t->size[d - 1] != 2 || t->stride[d - 1] != 1) return false;
  for (int i = 0; i < d - 1; ++i)
    if (t->stride[i] % 2 != 0) return false;
  return aligned(t->data, 8);
}

// [d0][d1][...][2] -> number of collapsed bins, or -1 if the middle dimensions
// are not one contiguous run of complex values
int collapsedBins(const fbfft_tensor* t) {
  const int d = t->dim;
  if (d < 3 || d > FBFFT_MAX_DIM) return -1;
  if (t->size[d - 1] != 2 || t->stride[d - 1] != 1) return -1;
  long expect = 2, xy = 1;
  for (int i = d - 2; i >= 2; --i) {
    if (t->size[i] != 1 && t->stride[i] != expect) return -1;
    expect *= t->size[i];
    xy *= t->size[i];
  }
  if (d == 3) xy = 1;  // [d0][d1][2]: a single bin
  return (int)xy;
}

// cplx[b][r][c] = 0 through the view's strides: the transform of an empty real
// window (all padding) is all zeros
__global__ void zeroSpectrum(CplxView v) {
  const long per = (long)v.rows * v.cols, total = per * v.B;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (long)gridDim.x * blockDim.x) {
    const long b = i / per, rc = i % per;
    float* p = v.data + b * v.sb + (rc / v.cols) * v.sr + (rc % v.cols) * v.sc;
    *reinterpret_cast<float2*>(p) = float2{0.0f, 0.0f};
  }
}

int launchZeroSpectrum(const CplxView& v, hipStream_t s) {
  const long total = (long)v.B * v.rows * v.cols;
  zeroSpectrum<<<dim3((unsigned)std::min<long>((total + 255) / 256, 8192)), 256, 0, s>>>(v);
  return launchStatus();
}

}  // namespace

extern "C" {

const char* fbfft_error_string(int code) {
  switch (code) {
    case FBFFT_SUCCESS: return "Success";
    case FBFFT_UNSUPPORTED_SIZE: return "UnsupportedSize";
    case FBFFT_UNSUPPORTED_DIMENSION: return "UnsupportedDimension";
    case FBFFT_HIP_ERROR: return "HipError";
  }
  return "Unknown";
}

void fbfft_twiddle_table(float* out) { memcpy(out, kTwiddleBits, sizeof(kTwiddleBits)); }

static int run1d(bool forward, const fbfft_tensor* real, const fbfft_tensor* cplx, int padL,
                 fbfft_stream_t stream) {
  if (!okTensor(real, 2) || !okTensor(cplx, 3)) return FBFFT_UNSUPPORTED_DIMENSION;
  const int N = real->size[1];
  if (!isPow2(N) || N < 2 || N > 256) return FBFFT_UNSUPPORTED_SIZE;
  if (cplx->size[2] != 2 || cplx->size[1] != N / 2 + 1 || cplx->size[0] != real->size[0])
    return FBFFT_UNSUPPORTED_DIMENSION;
  if (padL < 0) return FBFFT_UNSUPPORTED_SIZE;
  if (!okCplx(cplx)) return FBFFT_UNSUPPORTED_DIMENSION;
  if (real->size[0] == 0) return FBFFT_SUCCESS;
  return launchFft1d(forward, N, real->data, real->stride[0], real->stride[1], cplx->data,
                     cplx->stride[0], cplx->stride[1], real->size[0], padL, stream);
}

int fbfft_r2c_1d(const fbfft_tensor* real, const fbfft_tensor* cplx, int padL,
                 fbfft_stream_t stream) {
  return run1d(true, real, cplx, padL, stream);
}

int fbfft_c2r_1d(const fbfft_tensor* real, const fbfft_tensor* cplx, int padL,
                 fbfft_stream_t stream) {
  return run1d(false, real, cplx, padL, stream);
}

int fbfft_r2c_2d(const fbfft_tensor* real, const fbfft_tensor* cplx, int padL, int padU,
                 fbfft_stream_t stream) {
  if (!okTensor(real, 3) || !okTensor(cplx, 4)) return FBFFT_UNSUPPORTED_DIMENSION;
  if (cplx->size[3] != 2) return FBFFT_UNSUPPORTED_DIMENSION;
  if (real->size[0] != cplx->size[0]) return FBFFT_UNSUPPORTED_DIMENSION;
  const int s1 = cplx->size[1], s2 = cplx->size[2];
  int N = 0;
  bool scratchForm = false, packed = false;
  if ((s2 == 8 || s2 == 16 || s2 == 32) && s1 == s2 / 2) {
    N = s2;
    packed = true;
  } else if ((s2 == 2 || s2 == 4 || s2 == 8 || s2 == 16 || s2 == 32 || s2 == 64 || s2 == 128) &&
      s1 == s2 / 2 + 1) {
    N = s2;
  } else if ((s1 == 64 || s1 == 128) && s2 == s1 / 2 + 1) {
    N = s1;
    scratchForm = true;
  } else {
    return FBFFT_UNSUPPORTED_SIZE;
  }
  if (real->size[1] > N || real->size[2] > N || padL < 0 || padU < 0)
    return FBFFT_UNSUPPORTED_SIZE;
  if (!okCplx(cplx)) return FBFFT_UNSUPPORTED_DIMENSION;
  if (empty(cplx)) return FBFFT_SUCCESS;
  // B > 0 planes with an empty real window: every sample is padding
  if (empty(real)) return launchZeroSpectrum(cplxView4(cplx), stream);
  if (N < 8) return launchFft2dTinyForward(N, realView3(real), cplxView4(cplx), padL, padU, stream);
  if (N <= 32)
    return launchFft2dSmallForward(N, realView3(real), cplxView4(cplx), padL, padU, stream, packed);
  if (!scratchForm)
    return launchFft2dLargeForward(N, realView3(real), cplxView4(cplx), padL, padU, stream);
  return launchTwoPass(N, 0, real->data, real->stride[0], real->stride[1], real->stride[2],
                       cplx->data, cplx->stride[0], cplx->stride[1], cplx->stride[2],
                       real->size[0], real->size[1], real->size[2], padL, padU, stream);
}

int fbfft_c2r_2d(const fbfft_tensor* cplx, const fbfft_tensor* real, int padL, int padU,
                 fbfft_stream_t stream) {
  if (!okTensor(real, 3) || !okTensor(cplx, 4)) return FBFFT_UNSUPPORTED_DIMENSION;
  if (cplx->size[3] != 2) return FBFFT_UNSUPPORTED_DIMENSION;
  if (real->size[0] != cplx->size[0]) return FBFFT_UNSUPPORTED_DIMENSION;
  const int s1 = cplx->size[1], N = cplx->size[2];
  if (!(N == 2 || N == 4 || N == 8 || N == 16 || N == 32 || N == 64 || N == 128))
    return FBFFT_UNSUPPORTED_SIZE;
  const bool half = (s1 == N / 2 + 1);
  const bool full = (N >= 64 && s1 == N);
  const bool packed = (N >= 8 && N <= 32 && s1 == N / 2);
  if (!half && !full && !packed) return FBFFT_UNSUPPORTED_SIZE;
  if (padL < 0 || padU < 0) return FBFFT_UNSUPPORTED_SIZE;
  if (!okCplx(cplx)) return FBFFT_UNSUPPORTED_DIMENSION;
  if (empty(real) || empty(cplx)) return FBFFT_SUCCESS;
  if (N < 8) return launchFft2dTinyInverse(N, cplxView4(cplx), realView3(real), padL, padU, stream);
  if (N <= 32)
    return launchFft2dSmallInverse(N, cplxView4(cplx), realView3(real), padL, padU, stream, packed);
  if (half) return launchFft2dLargeInverse(N, cplxView4(cplx), realView3(real), padL, padU, stream);
  return launchTwoPass(N, 3, cplx->data, cplx->stride[0], cplx->stride[1], cplx->stride[2],
                       real->data, real->stride[0], real->stride[1], real->stride[2],
                       real->size[0], real->size[1], real->size[2], padL, padU, stream);
}

}  // extern "C"

extern "C" int fbfft_transpose_mm(const fbfft_tensor* A, const fbfft_tensor* B,
                                  const fbfft_tensor* C, int conjA, int conjB, int accumulate,
                                  float invNorm, fbfft_stream_t stream) {
  if (!A || !B || !C) return FBFFT_UNSUPPORTED_DIMENSION;
  if (conjA && conjB) return FBFFT_UNSUPPORTED_DIMENSION;  // no reference role uses both
  const int xa = collapsedBins(A), xb = collapsedBins(B), xc = collapsedBins(C);
  if (xa < 0 || xb < 0 || xc < 0 || xa != xb || xa != xc) return FBFFT_UNSUPPORTED_DIMENSION;
  const int I = conjA ? A->size[1] : A->size[0];
  const int K = conjA ? A->size[0] : A->size[1];
  const int Kb = conjB ? B->size[1] : B->size[0];
  const int J = conjB ? B->size[0] : B->size[1];
  if (K != Kb || C->size[0] != I || C->size[1] != J) return FBFFT_UNSUPPORTED_DIMENSION;
  const fbfft_tensor* ts[3] = {A, B, C};
  for (const fbfft_tensor* t : ts) {
    if (t->stride[0] % 2 != 0 || t->stride[1] % 2 != 0 || !aligned(t->data, 8))
      return FBFFT_UNSUPPORTED_DIMENSION;
  }
  return launchTransposeMM(A->data, A->stride[0], A->stride[1], B->data, B->stride[0],
                           B->stride[1], C->data, C->stride[0], C->stride[1], I, J, K, xa,
                           conjA != 0, conjB != 0, accumulate != 0, invNorm, stream);
}

extern "C" int fbfft_transpose_mm_packed(const fbfft_tensor* A, const fbfft_tensor* B,
                                         const fbfft_tensor* C, int conjA, int conjB,
                                         int accumulate, float invNorm, fbfft_stream_t stream) {
  if (!A || !B || !C) return FBFFT_UNSUPPORTED_DIMENSION;
  if (conjA && conjB) return FBFFT_UNSUPPORTED_DIMENSION;
  if (A->dim != 5 || B->dim != 5 || C->dim != 5) return FBFFT_UNSUPPORTED_DIMENSION;
  const int N = A->size[3];
  if (!(N == 8 || N == 16 || N == 32)) return FBFFT_UNSUPPORTED_SIZE;
  const fbfft_tensor* ts[3] = {A, B, C};
  for (const fbfft_tensor* t : ts) {
    if (t->size[3] != N || t->size[2] != N / 2) return FBFFT_UNSUPPORTED_SIZE;
    if (collapsedBins(t) != N / 2 * N) return FBFFT_UNSUPPORTED_DIMENSION;
    if (t->stride[0] % 2 != 0 || t->stride[1] % 2 != 0 || !aligned(t->data, 8))
      return FBFFT_UNSUPPORTED_DIMENSION;
  }
  const int I = conjA ? A->size[1] : A->size[0];
  const int K = conjA ? A->size[0] : A->size[1];
  const int Kb = conjB ? B->size[1] : B->size[0];
  const int J = conjB ? B->size[0] : B->size[1];
  if (K != Kb || C->size[0] != I || C->size[1] != J) return FBFFT_UNSUPPORTED_DIMENSION;
  return launchTransposeMMPacked(A->data, A->stride[0], A->stride[1], B->data, B->stride[0],
                                 B->stride[1], C->data, C->stride[0], C->stride[1], I, J, K, N,
                                 conjA != 0, conjB != 0, accumulate != 0, invNorm, stream);
}

namespace {

bool convSizeOk(int N) { return N == 8 || N == 16 || N == 32 || N == 64 || N == 128; }

// fftSize 0 in the layer entry points: the library's choice for the pass and the layer.
int resolveFftSize(int N, int pass, const fbfft_tensor* input, const fbfft_tensor* weight) {
  return N != 0 ? N
                : fbfft_conv_choose_fft_size(pass, input->size[0], input->size[1], weight->size[0],
                                             input->size[2], input->size[3], weight->size[2],
                                             weight->size[3]);
}

// Shapes of one convolution layer: input [B][Cin][H][W], weight [Cout][Cin][kH][kW],
// output [B][Cout][H-kH+1][W-kW+1], H, W <= N.
int checkConvShapes(int pass, const fbfft_tensor* input, const fbfft_tensor* weight,
                    const fbfft_tensor* output, int N) {
  if (!okTensor(input, 4) || !okTensor(weight, 4) || !okTensor(output, 4))
    return FBFFT_UNSUPPORTED_DIMENSION;
  N = resolveFftSize(N, pass, input, weight);
  if (!convSizeOk(N)) return FBFFT_UNSUPPORTED_SIZE;
  const int B = input->size[0], Cin = input->size[1], H = input->size[2], W = input->size[3];
  const int Cout = weight->size[0], kH = weight->size[2], kW = weight->size[3];
  if (weight->size[1] != Cin || output->size[0] != B || output->size[1] != Cout)
    return FBFFT_UNSUPPORTED_DIMENSION;
  if (kH > H || kW > W || kH > N || kW > N) return FBFFT_UNSUPPORTED_SIZE;
  // images larger than the transform are overlap-tiled by the 8 / 16 / 32-point path only
  if ((H > N || W > N) && N > 32) return FBFFT_UNSUPPORTED_SIZE;
  if (output->size[2] != H - kH + 1 || output->size[3] != W - kW + 1)
    return FBFFT_UNSUPPORTED_DIMENSION;
  return FBFFT_SUCCESS;
}

int convPass(int pass, const fbfft_tensor* input, const fbfft_tensor* weight,
             const fbfft_tensor* output, int N, float scale, bool accumulate, void* workspace,
             size_t workspaceBytes, fbfft_stream_t stream) {
  const int rc = checkConvShapes(pass, input, weight, output, N);
  if (rc != FBFFT_SUCCESS) return rc;
  if (empty(input) || empty(weight) || empty(output)) return FBFFT_SUCCESS;
  N = resolveFftSize(N, pass, input, weight);
  const size_t need = fbfft_conv_workspace_image(pass, input->size[0], input->size[1],
                                                 weight->size[0], input->size[2], input->size[3],
                                                 weight->size[2], weight->size[3], N);
  if (!workspace || !aligned(workspace, 256) || need == 0 || workspaceBytes < need)
    return FBFFT_UNSUPPORTED_DIMENSION;
  const fbfft_tensor *x, *y, *out;
  if (pass == 0) {
    x = input, y = weight, out = output;
  } else if (pass == 1) {
    x = output, y = weight, out = input;
  } else {
    x = input, y = output, out = weight;
  }
  return launchConvPass(pass, N, x->data, x->stride, x->size, y->data, y->stride, y->size,
                        out->data, out->stride, out->size, scale, accumulate, workspace, stream);
}

}  // namespace

extern "C" int fbfft_conv_choose_fft_size(int pass, int batch, int cin, int cout, int H, int W,
                                          int kH, int kW) {
  if (pass < 0 || pass > 2 || batch <= 0 || cin <= 0 || cout <= 0) return 0;
  if (kH < 1 || kW < 1 || kH > H || kW > W) return 0;
  // What a pass costs follows the spectrum values it moves: N^2 for every window of the
  // two image-sized tensors and for every filter plane.  The forward pass and the weight
  // gradient cut the OUTPUT into (N-kH+1) x (N-kW+1) windows, the input gradient cuts the
  // INPUT.  Smaller transforms run a little below the rate of 32-point ones (measured
  // over nine layer shapes: 1.15 x per value at 16 points, 1.5 x at 8), and their weight
  // gradients further below (1.25 x and 2 x: many windows make a long reduction over small
  // tiles).  The larger transform on a tie.  64 and 128 are never chosen: their layers run
  // plane-major spectra through transposeMM and measure slower than 32-point windows on
  // every shape tried.
  int best = 0;
  double bestCost = 0;
  for (int N = 8; N <= 32; N *= 2) {
    if (kH > N || kW > N) continue;
    const int spanY = pass == 1 ? H : H - kH + 1, spanX = pass == 1 ? W : W - kW + 1;
    // (an image that fits the transform is one window, whatever the pass: the rule of the
    // launcher's own window grid)
    const double tiles = (H <= N && W <= N)
                             ? 1.0
                             : (double)((spanY + N - kH) / (N - kH + 1)) * ((spanX + N - kW) / (N - kW + 1));
    const double values = (double)N * N * (tiles * batch * ((double)cin + cout) + (double)cin * cout);
    const double rate = N == 32 ? 1.0 : N == 16 ? (pass == 2 ? 1.25 : 1.15) : (pass == 2 ? 2.0 : 1.5);
    const double cost = values * rate;
    if (best == 0 || cost <= bestCost) {
      best = N;
      bestCost = cost;
    }
  }
  return best;
}

extern "C" size_t fbfft_conv_workspace_image(int pass, int batch, int cin, int cout, int H, int W,
                                             int kH, int kW, int fftSize) {
  if (pass < 0 || pass > 2 || batch <= 0 || cin <= 0 || cout <= 0) return 0;
  if (fftSize == 0) fftSize = fbfft_conv_choose_fft_size(pass, batch, cin, cout, H, W, kH, kW);
  if (!convSizeOk(fftSize)) return 0;
  if (kH < 1 || kW < 1 || kH > H || kW > W || kH > fftSize || kW > fftSize) return 0;
  if ((H > fftSize || W > fftSize) && fftSize > 32) return 0;
  return convWorkspaceBytes(pass, fftSize, batch, cin, cout, H, W, kH, kW);
}

extern "C" size_t fbfft_conv_workspace(int pass, int batch, int cin, int cout, int fftSize) {
  return fbfft_conv_workspace_image(pass, batch, cin, cout, fftSize, fftSize, 1, 1, fftSize);
}

extern "C" size_t fbfft_conv_fprop_workspace(int batch, int cin, int cout, int fftSize) {
  return fbfft_conv_workspace(0, batch, cin, cout, fftSize);
}

extern "C" int fbfft_conv_fprop(const fbfft_tensor* input, const fbfft_tensor* weight,
                                const fbfft_tensor* output, int fftSize, void* workspace,
                                size_t workspaceBytes, fbfft_stream_t stream) {
  return convPass(0, input, weight, output, fftSize, 1.0f, false, workspace, workspaceBytes,
                  stream);
}

extern "C" int fbfft_conv_bprop(const fbfft_tensor* gradOutput, const fbfft_tensor* weight,
                                const fbfft_tensor* gradInput, int fftSize, void* workspace,
                                size_t workspaceBytes, fbfft_stream_t stream) {
  return convPass(1, gradInput, weight, gradOutput, fftSize, 1.0f, false, workspace,
                  workspaceBytes, stream);
}

extern "C" int fbfft_conv_accgrad(const fbfft_tensor* input, const fbfft_tensor* gradOutput,
                                  const fbfft_tensor* gradWeight, int fftSize, float scale,
                                  int accumulate, void* workspace, size_t workspaceBytes,
                                  fbfft_stream_t stream) {
  return convPass(2, input, gradWeight, gradOutput, fftSize, scale, accumulate != 0, workspace,
                  workspaceBytes, stream);
}

extern "C" int fbfft_c2c_2d_pass2(const fbfft_tensor* src, const fbfft_tensor* dst,
                                  fbfft_stream_t stream) {
  if (!okTensor(src, 4) || !okTensor(dst, 4)) return FBFFT_UNSUPPORTED_DIMENSION;
  const int N = src->size[1];
  if (!(N == 64 || N == 128)) return FBFFT_UNSUPPORTED_SIZE;
  if (src->size[2] != N / 2 + 1 || dst->size[1] != N / 2 + 1 || dst->size[2] != N)
    return FBFFT_UNSUPPORTED_SIZE;
  if (src->size[0] != dst->size[0] || src->data == dst->data) return FBFFT_UNSUPPORTED_DIMENSION;
  if (!okCplx(src) || !okCplx(dst)) return FBFFT_UNSUPPORTED_DIMENSION;
  if (empty(src)) return FBFFT_SUCCESS;
  return launchTwoPass(N, 1, src->data, src->stride[0], src->stride[1], src->stride[2], dst->data,
                       dst->stride[0], dst->stride[1], dst->stride[2], src->size[0], 0, 0, 0, 0,
                       stream);
}

extern "C" int fbfft_c2c_2d_inverse_pass1(const fbfft_tensor* src, const fbfft_tensor* dst,
                                          fbfft_stream_t stream) {
  if (!okTensor(src, 4) || !okTensor(dst, 4)) return FBFFT_UNSUPPORTED_DIMENSION;
  const int N = src->size[2];
  // the size test of fbfft/FBIFFT2D-inl.cuh:537-542, narrowed to the sizes it dispatches
  if (!(N == 64 || N == 128) || src->size[1] != N / 2 + 1) return FBFFT_UNSUPPORTED_SIZE;
  if (dst->size[1] != N || dst->size[2] != N) return FBFFT_UNSUPPORTED_SIZE;
  if (dst->size[0] < (src->size[0] + 1) / 2) return FBFFT_UNSUPPORTED_DIMENSION;
  if (!okCplx(src) || !okCplx(dst)) return FBFFT_UNSUPPORTED_DIMENSION;
  if (empty(src)) return FBFFT_SUCCESS;
  return launchTwoPass(N, 2, src->data, src->stride[0], src->stride[1], src->stride[2], dst->data,
                       dst->stride[0], dst->stride[1], dst->stride[2], src->size[0], 0, 0, 0, 0,
                       stream);
}

extern "C" size_t fbfft_make_tiles_for_pass(int pass, const fbfft_tensor* input,
                                            const fbfft_tensor* output, int kH, int kW,
                                            int fftSize, fbfft_tile* ins, fbfft_tile* outs,
                                            size_t capacity) {
  if (!okTensor(input, 4) || !okTensor(output, 4)) return 0;
  if (pass < 0 || pass > 2) return 0;
  const int N = fftSize;
  if (!(N == 8 || N == 16 || N == 32) || kH < 1 || kW < 1 || kH > N || kW > N) return 0;
  const int H = input->size[2], W = input->size[3];
  const int oH = H - kH + 1, oW = W - kW + 1;
  if (oH < 1 || oW < 1 || output->size[2] != oH || output->size[3] != oW) return 0;
  if (output->size[0] != input->size[0]) return 0;
  const int stepY = N - kH + 1, stepX = N - kW + 1;
  // updateOutput / accGradParameters walk the output in disjoint step x step windows;
  // updateGradInput walks the input (the tensor it writes) in such windows
  const bool byInput = pass == FBFFT_UPDATE_GRAD_INPUT;
  const int spanY = byInput ? H : oH, spanX = byInput ? W : oW;
  const size_t ny = (size_t)ceilDiv(spanY, stepY), nx = (size_t)ceilDiv(spanX, stepX);
  if (!ins || !outs) return ny * nx;
  size_t n = 0;
  for (int y0 = 0; y0 < spanY; y0 += stepY) {
    for (int x0 = 0; x0 < spanX; x0 += stepX, ++n) {
      if (n >= capacity) continue;
      fbfft_tile& ti = ins[n];
      fbfft_tile& to = outs[n];
      for (int d = 0; d < 4; ++d) {
        ti.stride[d] = input->stride[d];
        to.stride[d] = output->stride[d];
      }
      ti.size[0] = input->size[0];
      ti.size[1] = input->size[1];
      to.size[0] = output->size[0];
      to.size[1] = output->size[1];
      int iy = y0, ix = x0, oy = y0, ox = x0;  // window origins in input / output
      if (!byInput) {
        ti.padL = ti.padU = to.padL = to.padU = 0;
        ti.size[2] = std::min(N, H - y0);
        ti.size[3] = std::min(N, W - x0);
        to.size[2] = std::min(stepY, oH - y0);
        to.size[3] = std::min(stepX, oW - x0);
      } else {
        // gradInput rows y0 .. y0+step-1 are a full convolution over gradOutput rows
        // y0-(kH-1) .. y0+step-1: N rows, placed from row 0 of the FFT plane (rows
        // above the tensor's first stay zero through padU, rows below its last through
        // the clipped size); the result for gradInput row y0 then sits in plane row
        // kH-1, clear of the circular wrap-around, which the destination's pads skip.
        oy = std::max(0, y0 - (kH - 1));
        ox = std::max(0, x0 - (kW - 1));
        to.padU = oy - (y0 - (kH - 1));
        to.padL = ox - (x0 - (kW - 1));
        to.size[2] = std::min(oH, y0 + stepY) - oy;
        to.size[3] = std::min(oW, x0 + stepX) - ox;
        ti.padU = kH - 1;
        ti.padL = kW - 1;
        ti.size[2] = std::min(stepY, H - y0);
        ti.size[3] = std::min(stepX, W - x0);
      }
      ti.data = input->data + (size_t)iy * input->stride[2] + (size_t)ix * input->stride[3];
      to.data = output->data + (size_t)oy * output->stride[2] + (size_t)ox * output->stride[3];
    }
  }
  return n;
}

extern "C" size_t fbfft_make_tiles(const fbfft_tensor* input, const fbfft_tensor* output, int kH,
                                   int kW, int fftSize, fbfft_tile* ins, fbfft_tile* outs,
                                   size_t capacity) {
  return fbfft_make_tiles_for_pass(FBFFT_UPDATE_OUTPUT, input, output, kH, kW, fftSize, ins, outs,
                                   capacity);
}

extern "C" size_t fbfft_iterated_conv_workspace(int fftSize, int pass, int batchSize,
                                               size_t numTiles, int cin, int cout) {
  if (!(fftSize == 8 || fftSize == 16 || fftSize == 32) || pass < 0 || pass > 2) return 0;
  if (batchSize <= 0 || numTiles == 0 || cin <= 0 || cout <= 0) return 0;
  if (numTiles > (size_t)1 << 30) return 0;
  return describedWorkspaceBytes(pass, fftSize, (long)numTiles * batchSize, cin, cout);
}

extern "C" int fbfft_iterated_conv_ws(int fftSize, const fbfft_tile* ins, const fbfft_tile* outs,
                                      const fbfft_tensor* weight, int pass, float scale,
                                      int batchSize, size_t numTiles, void* workspace,
                                      size_t workspaceBytes, fbfft_stream_t stream) {
  if (!okTensor(weight, 4) || !ins || !outs) return 0;
  if (!(fftSize == 8 || fftSize == 16 || fftSize == 32) || pass < 0 || pass > 2) return 0;
  if (weight->size[2] > fftSize || weight->size[3] > fftSize) return 0;
  if (batchSize <= 0 || numTiles == 0 || weight->size[0] <= 0 || weight->size[1] <= 0)
    return 1;  // nothing to do
  const size_t need = fbfft_iterated_conv_workspace(fftSize, pass, batchSize, numTiles,
                                                    weight->size[1], weight->size[0]);
  if (need == 0) return 0;
  if (!workspace || !aligned(workspace, 256) || workspaceBytes < need)
    return -FBFFT_UNSUPPORTED_DIMENSION;
  const int rc = launchDescribedConv(pass, fftSize, ins, outs, weight->data, weight->stride,
                                     weight->size, scale, batchSize, (int)numTiles, workspace,
                                     stream);
  return rc == FBFFT_SUCCESS ? 1 : -rc;
}

extern "C" int fbfft_iterated_conv(int fftSize, const fbfft_tile* ins, const fbfft_tile* outs,
                                   const fbfft_tensor* weight, int pass, float scale,
                                   int batchSize, size_t numTiles, fbfft_stream_t stream) {
  return fbfft_iterated_conv_ex(fftSize, ins, outs, weight, pass, scale, batchSize, numTiles, 0,
                                stream);
}

extern "C" int fbfft_iterated_conv_ex(int fftSize, const fbfft_tile* ins, const fbfft_tile* outs,
                                      const fbfft_tensor* weight, int pass, float scale,
                                      int batchSize, size_t numTiles, unsigned flags,
                                      fbfft_stream_t stream) {
  if (!okTensor(weight, 4) || !ins || !outs) return 0;
  if (flags & ~(unsigned)FBFFT_DETERMINISTIC) return 0;
  // a filter larger than the transform has no circular-convolution meaning; the
  // windowed loader would silently drop its rows / columns beyond fftSize
  if (weight->size[2] > fftSize || weight->size[3] > fftSize) return 0;
  return launchIteratedConv(fftSize, ins, outs, weight->data, weight->stride, weight->size, pass,
                            scale, batchSize, numTiles, (flags & FBFFT_DETERMINISTIC) != 0, stream);
}
