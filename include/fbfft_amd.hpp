// C++ facade over the C ABI of fbfft_amd.h: the reference's names, namespaces,
// template parameters and argument lists, so that host code written against
// fbcuda's fbfft headers compiles unchanged apart from the stream type
// (hipStream_t instead of cudaStream_t).  Header-only; link libfbfft_amd.so.
//
//   facebook::cuda::DeviceTensor<T, Dim>                  DeviceTensor.cuh:53-246 (host-side view only)
//   facebook::cuda::Complex                               Complex.cuh:16-140 (storage only)
//   facebook::cuda::fbfft::FBFFTParameters                fbfft/FBFFTParameters.h:7-59
//   facebook::cuda::fbfft::fbfft1D / fbifft1D / fbfft2D / fbifft2D   fbfft/FBFFT.cuh:11-56
//   facebook::cuda::transposeMM                           MM.cuh:11-17
//   facebook::cuda::fbfft::detail::TiledDeviceTensor, FFTConvolutionPassFFI,
//       FFTIteratedConvolution<N>                         fbfft/FFTIteratedConvolution.cuh:71-88, :616-755
#ifndef FBFFT_AMD_HPP
#define FBFFT_AMD_HPP

#include <cstddef>

#include "fbfft_amd.h"

namespace facebook { namespace cuda {

// Two packed floats, layout-compatible with the reference's cuComplex wrapper.
struct Complex {
  float re_, im_;
  Complex() : re_(0.f), im_(0.f) {}
  Complex(float r) : re_(r), im_(0.f) {}
  Complex(float r, float i) : re_(r), im_(i) {}
  float& re() { return re_; }
  float& im() { return im_; }
  const float& re() const { return re_; }
  const float& im() const { return im_; }
  Complex conjugate() const { return Complex(re_, -im_); }
  Complex transpose() const { return Complex(im_, re_); }
};
static_assert(sizeof(Complex) == 8, "Complex is two packed floats");

// Non-owning strided view with the reference's member order (data, strides,
// sizes); strides count elements of T.  Only what host code needs to describe an
// operand is provided: the kernels receive plain pointers and ints.
template <typename T, int Dim, typename IndexT = int>
class DeviceTensor {
 public:
  enum { NumDim = Dim };
  typedef T DataType;

  DeviceTensor() : data_(nullptr) {
    for (int i = 0; i < Dim; ++i) { stride_[i] = 0; size_[i] = 0; }
  }
  // contiguous, row-major
  DeviceTensor(T* data, const IndexT sizes[Dim]) : data_(data) {
    for (int i = 0; i < Dim; ++i) size_[i] = sizes[i];
    stride_[Dim - 1] = 1;
    for (int i = Dim - 2; i >= 0; --i) stride_[i] = stride_[i + 1] * size_[i + 1];
  }
  DeviceTensor(T* data, const IndexT sizes[Dim], const IndexT strides[Dim]) : data_(data) {
    for (int i = 0; i < Dim; ++i) { size_[i] = sizes[i]; stride_[i] = strides[i]; }
  }

  T* data() { return data_; }
  const T* data() const { return data_; }
  template <typename U> U* dataAs() { return reinterpret_cast<U*>(data_); }
  IndexT getSize(int i) const { return size_[i]; }
  IndexT getStride(int i) const { return stride_[i]; }
  const IndexT* sizes() const { return size_; }
  const IndexT* strides() const { return stride_; }

 private:
  T* data_;
  IndexT stride_[Dim];
  IndexT size_[Dim];
};

namespace fbfft_amd_detail {

template <int Dim>
inline fbfft_tensor describe(const DeviceTensor<float, Dim>& t) {
  static_assert(Dim <= FBFFT_MAX_DIM, "rank");
  fbfft_tensor d;
  d.data = const_cast<float*>(t.data());
  d.dim = Dim;
  for (int i = 0; i < FBFFT_MAX_DIM; ++i) {
    d.stride[i] = i < Dim ? t.getStride(i) : 0;
    d.size[i] = i < Dim ? t.getSize(i) : 0;
  }
  return d;
}

// a Complex tensor of rank Dim is a float tensor of rank Dim + 1 with a trailing [2]
template <int Dim>
inline fbfft_tensor describe(const DeviceTensor<Complex, Dim>& t) {
  static_assert(Dim + 1 <= FBFFT_MAX_DIM, "rank");
  fbfft_tensor d;
  d.data = reinterpret_cast<float*>(const_cast<Complex*>(t.data()));
  d.dim = Dim + 1;
  for (int i = 0; i < FBFFT_MAX_DIM; ++i) { d.stride[i] = 0; d.size[i] = 0; }
  for (int i = 0; i < Dim; ++i) {
    d.stride[i] = 2 * t.getStride(i);
    d.size[i] = t.getSize(i);
  }
  d.stride[Dim] = 1;
  d.size[Dim] = 2;
  return d;
}

}  // namespace fbfft_amd_detail

// The padding predicate of MemoryAccess.cuh:11-54: sample (y, x) of the padded
// plane lies inside the tensor's window placed at (padU, padL); one unsigned
// compare per axis tests both bounds.
inline bool inBounds(int x, int padL, const DeviceTensor<float, 2>& t) {
  return (unsigned)(x - padL) < (unsigned)t.getSize(1);
}
inline bool inBounds(int y, int x, int padU, int padL, const DeviceTensor<float, 3>& t) {
  return (unsigned)(y - padU) < (unsigned)t.getSize(1) &&
         (unsigned)(x - padL) < (unsigned)t.getSize(2);
}
inline bool inBounds(int y, int x, int padU, int padL, const DeviceTensor<float, 4>& t) {
  return (unsigned)(y - padU) < (unsigned)t.getSize(2) &&
         (unsigned)(x - padL) < (unsigned)t.getSize(3);
}
inline bool inBounds(int x, const DeviceTensor<float, 2>& t) {
  return (unsigned)x < (unsigned)t.getSize(1);
}

namespace fbfft {

// number of stored bins of a Hermitian half spectrum (FBFFTCommon.cuh:19-22)
template <typename T>
inline T numHermitian(T commonCols) {
  return commonCols / 2 + 1;
}

class FBFFTParameters {
 public:
  enum ErrorCode {
    Success = FBFFT_SUCCESS,
    UnsupportedSize = FBFFT_UNSUPPORTED_SIZE,
    UnsupportedDimension = FBFFT_UNSUPPORTED_DIMENSION,
    CudaError = FBFFT_HIP_ERROR,
    HipError = FBFFT_HIP_ERROR
  };

  FBFFTParameters& forward() { fwd_ = true; return *this; }
  FBFFTParameters& inverse() { fwd_ = false; return *this; }
  FBFFTParameters& normalize(bool n) { norm_ = n; return *this; }
  FBFFTParameters& withPadLeft(int p) { padL_ = p; return *this; }
  FBFFTParameters& withPadUp(int p) { padU_ = p; return *this; }

  bool forwardFFT() const { return fwd_; }
  bool inverseFFT() const { return !fwd_; }
  bool normalizeFFT() const { return norm_; }
  int padLeft() const { return padL_; }
  int padUp() const { return padU_; }

 private:
  bool fwd_ = true;
  bool norm_ = false;
  int padL_ = 0;
  int padU_ = 0;
};

namespace amd_detail {
inline FBFFTParameters::ErrorCode code(int rc) {
  return static_cast<FBFFTParameters::ErrorCode>(rc);
}
}  // namespace amd_detail

template <int BatchDims>
FBFFTParameters::ErrorCode fbfft1D(DeviceTensor<float, BatchDims + 1>& real,
                                   DeviceTensor<float, BatchDims + 2>& complex,
                                   const int padL = 0, fbfft_stream_t s = 0) {
  if (BatchDims != 1) return FBFFTParameters::UnsupportedDimension;
  fbfft_tensor r = fbfft_amd_detail::describe(real), c = fbfft_amd_detail::describe(complex);
  return amd_detail::code(fbfft_r2c_1d(&r, &c, padL, s));
}

template <int BatchDims>
FBFFTParameters::ErrorCode fbifft1D(DeviceTensor<float, BatchDims + 1>& real,
                                    DeviceTensor<float, BatchDims + 2>& complex,
                                    const int padL = 0, fbfft_stream_t s = 0) {
  if (BatchDims != 1) return FBFFTParameters::UnsupportedDimension;
  fbfft_tensor r = fbfft_amd_detail::describe(real), c = fbfft_amd_detail::describe(complex);
  return amd_detail::code(fbfft_c2r_1d(&r, &c, padL, s));
}

template <int BatchDims>
FBFFTParameters::ErrorCode fbfft2D(DeviceTensor<float, BatchDims + 2>& real,
                                   DeviceTensor<float, BatchDims + 3>& complex,
                                   const int padL = 0, const int padU = 0, fbfft_stream_t s = 0) {
  if (BatchDims != 1) return FBFFTParameters::UnsupportedDimension;
  fbfft_tensor r = fbfft_amd_detail::describe(real), c = fbfft_amd_detail::describe(complex);
  return amd_detail::code(fbfft_r2c_2d(&r, &c, padL, padU, s));
}

// second forward pass of the two-call form for N >= 64
template <int BatchDims>
FBFFTParameters::ErrorCode fbfft2D(DeviceTensor<Complex, BatchDims + 2>& src,
                                   DeviceTensor<Complex, BatchDims + 2>& dst,
                                   fbfft_stream_t s = 0) {
  if (BatchDims != 1) return FBFFTParameters::UnsupportedDimension;
  fbfft_tensor a = fbfft_amd_detail::describe(src), b = fbfft_amd_detail::describe(dst);
  return amd_detail::code(fbfft_c2c_2d_pass2(&a, &b, s));
}

// first inverse pass of the two-call form for N >= 64
template <int BatchDims>
FBFFTParameters::ErrorCode fbifft2D(DeviceTensor<float, BatchDims + 3>& src,
                                    DeviceTensor<float, BatchDims + 3>& dst,
                                    fbfft_stream_t s = 0) {
  if (BatchDims != 1) return FBFFTParameters::UnsupportedDimension;
  fbfft_tensor a = fbfft_amd_detail::describe(src), b = fbfft_amd_detail::describe(dst);
  return amd_detail::code(fbfft_c2c_2d_inverse_pass1(&a, &b, s));
}

template <int BatchDims>
FBFFTParameters::ErrorCode fbifft2D(DeviceTensor<Complex, BatchDims + 2>& complexSrc,
                                    DeviceTensor<float, BatchDims + 2>& realDst,
                                    const int padL = 0, const int padU = 0,
                                    fbfft_stream_t s = 0) {
  if (BatchDims != 1) return FBFFTParameters::UnsupportedDimension;
  fbfft_tensor c = fbfft_amd_detail::describe(complexSrc), r = fbfft_amd_detail::describe(realDst);
  return amd_detail::code(fbfft_c2r_2d(&c, &r, padL, padU, s));
}

namespace detail {

template <typename T, int Dims>
struct TiledDeviceTensor {
  TiledDeviceTensor() : padL(-1), padU(-1), tensor() {}
  TiledDeviceTensor(DeviceTensor<T, Dims>& t, int leftPadding, int upPadding)
      : padL(leftPadding), padU(upPadding), tensor(t.data(), t.sizes(), t.strides()) {}
  int padL;
  int padU;
  DeviceTensor<T, Dims> tensor;
};
static_assert(sizeof(TiledDeviceTensor<float, 4>) == sizeof(fbfft_tile),
              "descriptor layout must match the C ABI");

typedef struct _FFTConvolutionPassFFI {
  static const int FFT_UpdateOutput = FBFFT_UPDATE_OUTPUT;
  static const int FFT_UpdateGradInput = FBFFT_UPDATE_GRAD_INPUT;
  static const int FFT_AccGradParameters = FBFFT_ACC_GRAD_PARAMETERS;
  int pass;
} FFTConvolutionPassFFI;

// ins / outs: device pointers to numTiles descriptors
template <int FFTSize>
bool FFTIteratedConvolution(TiledDeviceTensor<float, 4>* ins, TiledDeviceTensor<float, 4>* outs,
                            const DeviceTensor<float, 4> weight, FFTConvolutionPassFFI pass,
                            float scale, int batchSize, size_t numTiles, fbfft_stream_t s) {
  fbfft_tensor w = fbfft_amd_detail::describe(weight);
  return fbfft_iterated_conv(FFTSize, reinterpret_cast<const fbfft_tile*>(ins),
                             reinterpret_cast<const fbfft_tile*>(outs), &w, pass.pass, scale,
                             batchSize, numTiles, s) == 1;
}

// Host-side tile grid for FFTIteratedConvolution<FFTSize>: fills ins / outs (host
// arrays of capacity descriptors) and returns the tile count; see
// fbfft_make_tiles_for_pass.  FFT_UpdateGradInput needs its own grid (disjoint
// gradInput windows); the other two passes share one.
template <int FFTSize>
size_t makeTiles(const DeviceTensor<float, 4>& input, const DeviceTensor<float, 4>& output, int kH,
                 int kW, TiledDeviceTensor<float, 4>* ins, TiledDeviceTensor<float, 4>* outs,
                 size_t capacity,
                 FFTConvolutionPassFFI pass = FFTConvolutionPassFFI{FBFFT_UPDATE_OUTPUT}) {
  fbfft_tensor i = fbfft_amd_detail::describe(input), o = fbfft_amd_detail::describe(output);
  return fbfft_make_tiles_for_pass(pass.pass, &i, &o, kH, kW, FFTSize,
                                   reinterpret_cast<fbfft_tile*>(ins),
                                   reinterpret_cast<fbfft_tile*>(outs), capacity);
}

}  // namespace detail
}  // namespace fbfft

template <int Dim, bool ConjugateTransposeA, bool ConjugateTransposeB, bool Accumulate>
void transposeMM(DeviceTensor<float, Dim>& A, DeviceTensor<float, Dim>& B,
                 DeviceTensor<float, Dim>& C, float invNorm, fbfft_stream_t s = 0) {
  fbfft_tensor a = fbfft_amd_detail::describe(A), b = fbfft_amd_detail::describe(B),
               c = fbfft_amd_detail::describe(C);
  fbfft_transpose_mm(&a, &b, &c, ConjugateTransposeA, ConjugateTransposeB, Accumulate, invNorm, s);
}

// The three passes of a convolution layer on the split FFT -> transposeMM -> IFFT
// path, which the reference's external callers compose themselves
// (MM-inl.cuh:188-196).  workspace: device memory of fftConvolutionWorkspace bytes.
namespace fbfft {

inline size_t fftConvolutionWorkspace(detail::FFTConvolutionPassFFI pass, int batch, int cin,
                                      int cout, int fftSize) {
  return fbfft_conv_workspace(pass.pass, batch, cin, cout, fftSize);
}

inline FBFFTParameters::ErrorCode fftConvolutionUpdateOutput(
    DeviceTensor<float, 4>& input, DeviceTensor<float, 4>& weight, DeviceTensor<float, 4>& output,
    int fftSize, void* workspace, size_t workspaceBytes, fbfft_stream_t s = 0) {
  fbfft_tensor i = fbfft_amd_detail::describe(input), w = fbfft_amd_detail::describe(weight),
               o = fbfft_amd_detail::describe(output);
  return amd_detail::code(fbfft_conv_fprop(&i, &w, &o, fftSize, workspace, workspaceBytes, s));
}

inline FBFFTParameters::ErrorCode fftConvolutionUpdateGradInput(
    DeviceTensor<float, 4>& gradOutput, DeviceTensor<float, 4>& weight,
    DeviceTensor<float, 4>& gradInput, int fftSize, void* workspace, size_t workspaceBytes,
    fbfft_stream_t s = 0) {
  fbfft_tensor g = fbfft_amd_detail::describe(gradOutput), w = fbfft_amd_detail::describe(weight),
               i = fbfft_amd_detail::describe(gradInput);
  return amd_detail::code(fbfft_conv_bprop(&g, &w, &i, fftSize, workspace, workspaceBytes, s));
}

inline FBFFTParameters::ErrorCode fftConvolutionAccGradParameters(
    DeviceTensor<float, 4>& input, DeviceTensor<float, 4>& gradOutput,
    DeviceTensor<float, 4>& gradWeight, int fftSize, float scale, bool accumulate, void* workspace,
    size_t workspaceBytes, fbfft_stream_t s = 0) {
  fbfft_tensor i = fbfft_amd_detail::describe(input), g = fbfft_amd_detail::describe(gradOutput),
               w = fbfft_amd_detail::describe(gradWeight);
  return amd_detail::code(fbfft_conv_accgrad(&i, &g, &w, fftSize, scale, accumulate, workspace,
                                             workspaceBytes, s));
}

}  // namespace fbfft


} }  // namespace facebook::cuda

#endif  // FBFFT_AMD_HPP
