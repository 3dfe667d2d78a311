// C++ facade over the C ABI of fbfft_amd.h: the reference's names, namespaces,
// template parameters and argument lists, so that host code written against
// fbcuda's fbfft headers compiles unchanged apart from the stream type
// (hipStream_t instead of cudaStream_t).  Header-only; link libfbfft_amd.so.
//
//   facebook::cuda::DeviceTensor<T, Dim>                  DeviceTensor.cuh:53-246 (the host-side interface)
//   facebook::cuda::Complex                               Complex.cuh:16-140
//   facebook::cuda::fbfft::FBFFTParameters                fbfft/FBFFTParameters.h:7-59
//   facebook::cuda::fbfft::fbfft1D / fbifft1D / fbfft2D / fbifft2D   fbfft/FBFFT.cuh:11-56
//   facebook::cuda::transposeMM                           MM.cuh:11-17
//   facebook::cuda::fbfft::detail::TiledDeviceTensor, FFTConvolutionPassFFI,
//       FFTIteratedConvolution<N>                         fbfft/FFTIteratedConvolution.cuh:71-88, :616-755
#ifndef FBFFT_AMD_HPP
#define FBFFT_AMD_HPP

#include <cmath>
#include <cstddef>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "fbfft_amd.h"

namespace facebook { namespace cuda {

// Two packed floats, layout-compatible with the reference's cuComplex wrapper
// (Complex.cuh:16-140), with its host-side arithmetic: products and quotients follow
// cuComplex.h (cuCmulf: (ac - bd, ad + bc); cuCdivf: both operands scaled by
// 1 / (|c| + |d|) before the division).
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
  void cexp(float angle) { re_ = std::cos(angle); im_ = std::sin(angle); }

  bool operator==(const Complex& o) const { return re_ == o.re_ && im_ == o.im_; }
  bool operator!=(const Complex& o) const { return !(*this == o); }
  Complex operator-() const { return Complex(-re_, -im_); }
  Complex operator+(const Complex& o) const { return Complex(re_ + o.re_, im_ + o.im_); }
  Complex operator-(const Complex& o) const { return Complex(re_ - o.re_, im_ - o.im_); }
  Complex operator*(const Complex& o) const {
    return Complex(re_ * o.re_ - im_ * o.im_, re_ * o.im_ + im_ * o.re_);
  }
  Complex operator/(const Complex& o) const {
    const float scale = 1.0f / (std::fabs(o.re_) + std::fabs(o.im_));
    const float ar = re_ * scale, ai = im_ * scale, br = o.re_ * scale, bi = o.im_ * scale;
    const float inv = 1.0f / (br * br + bi * bi);
    return Complex((ar * br + ai * bi) * inv, (ai * br - ar * bi) * inv);
  }
  Complex& operator+=(const Complex& o) { return *this = *this + o; }
  Complex& operator-=(const Complex& o) { return *this = *this - o; }
  Complex& operator*=(const Complex& o) { return *this = *this * o; }
  Complex& operator/=(const Complex& o) { return *this = *this / o; }
};
static_assert(sizeof(Complex) == 8, "Complex is two packed floats");

template <typename T, int Dim, typename IndexT>
class DeviceTensor;

namespace fbfft_amd_detail {

// tensor[i][j]...: the address arithmetic of the reference's DeviceSubTensor
// (DeviceTensor.cuh:249-379) for host code, which can only take addresses of
// device memory: data() of the indexed element or sub-tensor.
template <typename T, int Left, typename IndexT>
class SubView {
 public:
  SubView(T* at, const IndexT* strides) : at_(at), strides_(strides) {}
  SubView<T, Left - 1, IndexT> operator[](IndexT i) const {
    static_assert(Left >= 1, "too many indices");
    return SubView<T, Left - 1, IndexT>(at_ + (std::ptrdiff_t)i * strides_[0], strides_ + 1);
  }
  T* data() const { return at_; }

 private:
  T* at_;
  const IndexT* strides_;
};

}  // namespace fbfft_amd_detail

// Non-owning strided view with the reference's member order (data, strides,
// sizes) and its host-side interface (DeviceTensor.cuh:53-246,
// DeviceTensor-inl.cuh); strides count elements of T.  Everything here is size /
// stride arithmetic on the host: the kernels receive plain pointers and ints.
// Invariant violations throw std::invalid_argument, as the reference's host code does.
template <typename T, int Dim, typename IndexT = int>
class DeviceTensor {
 public:
  enum { NumDim = Dim };
  typedef T DataType;
  typedef IndexT IndexType;
  typedef T* DataPtrType;
  typedef DeviceTensor<T, Dim, IndexT> TensorType;
  static_assert(Dim > 0, "rank");

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
  template <typename U> const U* dataAs() const { return reinterpret_cast<const U*>(data_); }
  IndexT getSize(int i) const { return size_[i]; }
  IndexT getStride(int i) const { return stride_[i]; }
  const IndexT* sizes() const { return size_; }
  const IndexT* strides() const { return stride_; }

  fbfft_amd_detail::SubView<T, Dim - 1, IndexT> operator[](IndexT i) const {
    return fbfft_amd_detail::SubView<T, Dim - 1, IndexT>(data_ + (std::ptrdiff_t)i * stride_[0],
                                                         stride_ + 1);
  }

  template <int OtherDim>
  bool isSameSize(const DeviceTensor<T, OtherDim, IndexT>& rhs) const {
    if (Dim != OtherDim) return false;
    for (int i = 0; i < Dim; ++i)
      if (size_[i] != rhs.getSize(i)) return false;
    return true;
  }
  template <int OtherDim>
  bool isSameSizeAndStride(const DeviceTensor<T, OtherDim, IndexT>& rhs) const {
    if (!isSameSize(rhs)) return false;
    for (int i = 0; i < Dim; ++i)
      if (stride_[i] != rhs.getStride(i)) return false;
    return true;
  }

  // "sizes: [a, b]  strides: [c, d]"
  std::string toString() const {
    auto list = [](const IndexT* v) {
      std::string out = "[";
      for (int i = 0; i < Dim; ++i) out += (i ? ", " : "") + std::to_string(v[i]);
      return out + "]";
    };
    return "sizes: " + list(size_) + "  strides: " + list(stride_);
  }

  // the same view on elements of another type of the same width
  template <typename U>
  DeviceTensor<U, Dim, IndexT> cast() const {
    static_assert(sizeof(U) == sizeof(T), "cast keeps the element width");
    return DeviceTensor<U, Dim, IndexT>(reinterpret_cast<U*>(data_), size_, stride_);
  }

  long numElements() const {
    long n = 1;
    for (int i = 0; i < Dim; ++i) n *= size_[i];
    return n;
  }

  // dimension i directly encloses dimension i + 1 (no padding between them)
  bool isContiguousDim(int i) const {
    if (i == Dim - 1) return true;
    return i >= 0 && i < Dim - 1 && stride_[i] / stride_[i + 1] == size_[i + 1];
  }
  // dense row-major, dimensions of size 1 aside
  bool isContiguous() const {
    long expect = 1;
    for (int i = Dim - 1; i >= 0; --i) {
      if (size_[i] == 1) continue;
      if (stride_[i] != expect) return false;
      expect *= size_[i];
    }
    return true;
  }
  // stride positive and, for i > 0, no larger extent than the enclosing stride allows
  bool isConsistentlySized(int i) const {
    if (i < 0 || i >= Dim || stride_[i] <= 0) return false;
    return i == 0 ? size_[0] > 0 : stride_[i - 1] / stride_[i] >= size_[i];
  }
  bool isConsistentlySized() const {
    for (int i = 0; i < Dim; ++i)
      if (!isConsistentlySized(i)) return false;
    return true;
  }

  // Reorders the SIZES by perm and recomputes dense strides (the data is not moved);
  // dense tensors only.
  void permuteDims(const std::vector<int>& perm) {
    if ((int)perm.size() != Dim)
      throw std::invalid_argument("Permutation list must be of the same size as our dimension");
    if (stride_[Dim - 1] != 1) throw std::invalid_argument("Innermost dimension must have stride 1");
    for (int i = 0; i < Dim; ++i)
      if (!isContiguousDim(i)) throw std::invalid_argument("All dimensions must be contiguous");
    IndexT sz[Dim];
    for (int i = 0; i < Dim; ++i) sz[i] = size_[perm[i]];
    *this = DeviceTensor(data_, sz);
  }

  // sizes and strides of two dimensions exchanged; no data movement
  DeviceTensor transpose(int dim1, int dim2) const {
    if (dim1 < 0 || dim1 >= Dim) throw std::invalid_argument("dim1 out of bounds");
    if (dim2 < 0 || dim2 >= Dim) throw std::invalid_argument("dim2 out of bounds");
    DeviceTensor t = *this;
    std::swap(t.size_[dim1], t.size_[dim2]);
    std::swap(t.stride_[dim1], t.stride_[dim2]);
    return t;
  }

  // [2][3] -> [1][1][2][3]; the new dimensions stride over the whole tensor
  template <int NewDim>
  DeviceTensor<T, NewDim, IndexT> upcastOuter() const {
    static_assert(NewDim > Dim, "upcast raises the rank");
    IndexT sz[NewDim], st[NewDim];
    for (int i = 0; i < NewDim - Dim; ++i) { sz[i] = 1; st[i] = size_[0] * stride_[0]; }
    for (int i = 0; i < Dim; ++i) { sz[NewDim - Dim + i] = size_[i]; st[NewDim - Dim + i] = stride_[i]; }
    return DeviceTensor<T, NewDim, IndexT>(data_, sz, st);
  }
  // [2][3] -> [2][3][1][1]
  template <int NewDim>
  DeviceTensor<T, NewDim, IndexT> upcastInner() const {
    static_assert(NewDim > Dim, "upcast raises the rank");
    IndexT sz[NewDim], st[NewDim];
    for (int i = 0; i < NewDim; ++i) { sz[i] = i < Dim ? size_[i] : 1; st[i] = i < Dim ? stride_[i] : 1; }
    return DeviceTensor<T, NewDim, IndexT>(data_, sz, st);
  }
  // [a][b][c][d] -> [a*b*c][d] for NewDim = 2: the leading dimensions collapse into
  // the first one kept; they must enclose each other without padding
  template <int NewDim>
  DeviceTensor<T, NewDim, IndexT> downcastOuter() const {
    static_assert(NewDim < Dim, "downcast lowers the rank");
    constexpr int gone = Dim - NewDim;
    IndexT sz[NewDim], st[NewDim];
    IndexT lead = 1;
    for (int i = 0; i < gone; ++i) {
      if (!isContiguousDim(i)) throw std::invalid_argument("Can only downcast contiguous tensors");
      lead *= size_[i];
    }
    for (int i = 0; i < NewDim; ++i) { sz[i] = size_[gone + i]; st[i] = stride_[gone + i]; }
    sz[0] *= lead;
    return DeviceTensor<T, NewDim, IndexT>(data_, sz, st);
  }
  // [a][b][c][d] -> [a][b*c*d] for NewDim = 2: the trailing dimensions collapse into
  // the last one kept, which takes the innermost stride
  template <int NewDim>
  DeviceTensor<T, NewDim, IndexT> downcastInner() const {
    static_assert(NewDim < Dim, "downcast lowers the rank");
    IndexT sz[NewDim], st[NewDim];
    IndexT tail = 1;
    for (int i = NewDim; i < Dim; ++i) {
      if (!isContiguousDim(i)) throw std::invalid_argument("Can only downcast contiguous tensors");
      tail *= size_[i];
    }
    for (int i = 0; i < NewDim; ++i) { sz[i] = size_[i]; st[i] = stride_[i]; }
    sz[NewDim - 1] *= tail;
    st[NewDim - 1] = stride_[Dim - 1];
    return DeviceTensor<T, NewDim, IndexT>(data_, sz, st);
  }
  // the innermost SubDim dimensions as a tensor starting at `at`
  template <int SubDim>
  DeviceTensor<T, SubDim, IndexT> view(T* at) const {
    static_assert(SubDim >= 1 && SubDim < Dim, "a view has lower rank");
    return DeviceTensor<T, SubDim, IndexT>(at, size_ + (Dim - SubDim), stride_ + (Dim - SubDim));
  }
  template <int SubDim>
  DeviceTensor<T, SubDim, IndexT> view() const {
    return view<SubDim>(data_);
  }

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

// ins / outs: device pointers to numTiles descriptors.  deterministic (not in the
// reference's signature): FFT_AccGradParameters reduces in the reference's fixed order,
// reproducible bit for bit and much slower; see fbfft_iterated_conv_ex.
template <int FFTSize>
bool FFTIteratedConvolution(TiledDeviceTensor<float, 4>* ins, TiledDeviceTensor<float, 4>* outs,
                            const DeviceTensor<float, 4> weight, FFTConvolutionPassFFI pass,
                            float scale, int batchSize, size_t numTiles, fbfft_stream_t s,
                            bool deterministic = false) {
  fbfft_tensor w = fbfft_amd_detail::describe(weight);
  return fbfft_iterated_conv_ex(FFTSize, reinterpret_cast<const fbfft_tile*>(ins),
                                reinterpret_cast<const fbfft_tile*>(outs), &w, pass.pass, scale,
                                batchSize, numTiles, deterministic ? FBFFT_DETERMINISTIC : 0u,
                                s) == 1;
}

// The same call for callers that can lend a workspace (not in the reference's
// signature): the same descriptors and results, computed by the kernels of the
// convolution layer entry points instead of the fused kernel - about twice as fast at
// configs[4] - with a weight gradient that is reproducible bit for bit; see
// fbfft_iterated_conv_ws.  workspaceBytes >= iteratedConvolutionWorkspace<FFTSize>(...).
template <int FFTSize>
size_t iteratedConvolutionWorkspace(const DeviceTensor<float, 4>& weight, FFTConvolutionPassFFI pass,
                                    int batchSize, size_t numTiles) {
  return fbfft_iterated_conv_workspace(FFTSize, pass.pass, batchSize, numTiles, weight.getSize(1),
                                       weight.getSize(0));
}

template <int FFTSize>
bool FFTIteratedConvolution(TiledDeviceTensor<float, 4>* ins, TiledDeviceTensor<float, 4>* outs,
                            const DeviceTensor<float, 4> weight, FFTConvolutionPassFFI pass,
                            float scale, int batchSize, size_t numTiles, void* workspace,
                            size_t workspaceBytes, fbfft_stream_t s) {
  fbfft_tensor w = fbfft_amd_detail::describe(weight);
  return fbfft_iterated_conv_ws(FFTSize, reinterpret_cast<const fbfft_tile*>(ins),
                                reinterpret_cast<const fbfft_tile*>(outs), &w, pass.pass, scale,
                                batchSize, numTiles, workspace, workspaceBytes, s) == 1;
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

// transposeMM on spectra in the packed format of fbfft2D (DeviceTensor<float, 5>
// [d0][d1][N/2][N][2], N in {8,16,32}; fbfft/FFT2D32.cuh:421-427 declares the
// format, the reference ships no contraction for it): see fbfft_transpose_mm_packed.
template <bool ConjugateTransposeA, bool ConjugateTransposeB, bool Accumulate>
fbfft::FBFFTParameters::ErrorCode transposeMMPacked(DeviceTensor<float, 5>& A, DeviceTensor<float, 5>& B,
                                             DeviceTensor<float, 5>& C, float invNorm,
                                             fbfft_stream_t s = 0) {
  fbfft_tensor a = fbfft_amd_detail::describe(A), b = fbfft_amd_detail::describe(B),
               c = fbfft_amd_detail::describe(C);
  return (fbfft::FBFFTParameters::ErrorCode)fbfft_transpose_mm_packed(
      &a, &b, &c, ConjugateTransposeA, ConjugateTransposeB, Accumulate, invNorm, s);
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
