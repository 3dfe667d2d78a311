// C ABI: argument validation and dispatch.  Nothing here touches device memory
// or synchronises; every kernel is enqueued on the caller's stream.
#include <string.h>

#include "common.h"
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

int fbfft_r2c_2d(const fbfft_tensor* real, const fbfft_tensor* cplx, int padL, int padU,
                 fbfft_stream_t stream) {
  if (!okTensor(real, 3) || !okTensor(cplx, 4)) return FBFFT_UNSUPPORTED_DIMENSION;
  if (cplx->size[3] != 2) return FBFFT_UNSUPPORTED_DIMENSION;
  if (real->size[0] != cplx->size[0]) return FBFFT_UNSUPPORTED_DIMENSION;
  const int s1 = cplx->size[1], s2 = cplx->size[2];
  int N = 0;
  bool scratchForm = false;
  if ((s2 == 8 || s2 == 16 || s2 == 32 || s2 == 64 || s2 == 128) && s1 == s2 / 2 + 1) {
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
  if (empty(real) || empty(cplx)) return FBFFT_SUCCESS;
  if (N <= 32) return launchFft2dSmallForward(N, realView3(real), cplxView4(cplx), padL, padU, stream);
  if (!scratchForm)
    return launchFft2dLargeForward(N, realView3(real), cplxView4(cplx), padL, padU, stream);
  return FBFFT_UNSUPPORTED_SIZE;
}

int fbfft_c2r_2d(const fbfft_tensor* cplx, const fbfft_tensor* real, int padL, int padU,
                 fbfft_stream_t stream) {
  if (!okTensor(real, 3) || !okTensor(cplx, 4)) return FBFFT_UNSUPPORTED_DIMENSION;
  if (cplx->size[3] != 2) return FBFFT_UNSUPPORTED_DIMENSION;
  if (real->size[0] != cplx->size[0]) return FBFFT_UNSUPPORTED_DIMENSION;
  const int s1 = cplx->size[1], N = cplx->size[2];
  if (!(N == 8 || N == 16 || N == 32 || N == 64 || N == 128)) return FBFFT_UNSUPPORTED_SIZE;
  const bool half = (s1 == N / 2 + 1);
  const bool full = (N >= 64 && s1 == N);
  if (!half && !full) return FBFFT_UNSUPPORTED_SIZE;
  if (padL < 0 || padU < 0) return FBFFT_UNSUPPORTED_SIZE;
  if (!okCplx(cplx)) return FBFFT_UNSUPPORTED_DIMENSION;
  if (empty(real) || empty(cplx)) return FBFFT_SUCCESS;
  if (N <= 32) return launchFft2dSmallInverse(N, cplxView4(cplx), realView3(real), padL, padU, stream);
  if (half) return launchFft2dLargeInverse(N, cplxView4(cplx), realView3(real), padL, padU, stream);
  return FBFFT_UNSUPPORTED_SIZE;
}

}  // extern "C"

// ---- entry points whose kernels are not wired yet ----
extern "C" {
int fbfft_r2c_1d(const fbfft_tensor*, const fbfft_tensor*, int, fbfft_stream_t) { return FBFFT_UNSUPPORTED_SIZE; }
int fbfft_c2r_1d(const fbfft_tensor*, const fbfft_tensor*, int, fbfft_stream_t) { return FBFFT_UNSUPPORTED_SIZE; }
int fbfft_c2c_2d_pass2(const fbfft_tensor*, const fbfft_tensor*, fbfft_stream_t) { return FBFFT_UNSUPPORTED_SIZE; }
int fbfft_c2c_2d_inverse_pass1(const fbfft_tensor*, const fbfft_tensor*, fbfft_stream_t) { return FBFFT_UNSUPPORTED_SIZE; }
int fbfft_transpose_mm(const fbfft_tensor*, const fbfft_tensor*, const fbfft_tensor*, int, int, int, float, fbfft_stream_t) { return FBFFT_UNSUPPORTED_SIZE; }
int fbfft_iterated_conv(int, const fbfft_tile*, const fbfft_tile*, const fbfft_tensor*, int, float, int, size_t, fbfft_stream_t) { return 0; }
size_t fbfft_conv_fprop_workspace(int, int, int, int) { return 0; }
int fbfft_conv_fprop(const fbfft_tensor*, const fbfft_tensor*, const fbfft_tensor*, int, void*, size_t, fbfft_stream_t) { return FBFFT_UNSUPPORTED_SIZE; }
}
